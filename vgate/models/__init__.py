"""Model families and the registry that maps an architecture to its model class."""
from __future__ import annotations


def build_model(arch, device, tp=None, quantization=None, seed: int = 0, weights_path: str | None = None,
                max_model_len: int = 4096, dtype: str = "bfloat16"):
    """Instantiate the model class of ``arch.family`` (weights loaded from ``weights_path`` or
    random-initialised from ``seed``)."""
    from vgate.models.hybrid import HybridModel
    from vgate.models.transformer import DecoderModel
    registry = {"qwen2": DecoderModel, "llama": DecoderModel, "zadirax": HybridModel}
    cls = registry.get(arch.family)
    if cls is None:
        raise ValueError(f"no model class for family {arch.family!r} (known: {sorted(registry)})")
    dtype = {"auto": "bfloat16", "bf16": "bfloat16", "fp32": "float32"}.get(dtype, dtype)
    if cls is DecoderModel:
        if dtype == "float32":
            raise ValueError(f"the {arch.family} family runs in bfloat16 only (dtype {dtype!r} asked)")
        return DecoderModel(arch, device, tp, quantization, seed, weights_path, max_model_len)
    return cls(arch, device, tp, quantization, seed, weights_path, max_model_len, dtype=dtype)
