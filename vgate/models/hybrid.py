"""Layered hybrid decoder: a list of layers, each a token mixer (``vgate.models.mixers.MIXERS``) and
an optional feed-forward, over an fp32 residual stream.

One forward pass = one engine step over a flat token batch (any mix of prompt portions and single
decoded tokens) with all step metadata in device buffers (:class:`vgate.runtime.step_meta.StepView`),
as for the transformer families, so the same code is captured into a hipGraph per bucket.

Layer (parallel arrangement, gated residual):
    h  = x / sqrt(mean(x^2) + eps) * g            one scalar weight per norm; h in the activation dtype
    P  = h @ [mixer inputs; rg1; rg2]^T           ONE fused input projection per layer
    x += mixer(h) * sigmoid(P_rg1 + b1) + ff(h) * sigmoid(P_rg2 + b2)
A layer may run with another layer's weights (``weights_of``) while keeping its own cache or state.
Activation dtype bf16 (MFMA GEMMs, fp32 accumulation) or fp32 (true fp32 FMA everywhere); the residual
stream, norms, scores, routers and recurrent state are fp32 in both.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch

from vgate.models.config import HybridArch
from vgate.models.mixers import FEED_FORWARDS, MIXERS, Proj, _f32, _pad8, layer_shapes
from vgate.ops import seq
from vgate.parallel.comm import TPGroup


class LayerWeights:
    """The tensors of one weight-owning layer in kernel-ready form."""

    def __init__(self, spec, width: int, eps: float, t: dict, device, f32: bool):
        mix = {k[4:]: v for k, v in t.items() if k.startswith("mix.")}
        self.mixer = MIXERS[spec.kind](spec.mixer, width, eps, mix, device, f32)
        self.ff = None
        if spec.mlp:
            mlp = {k[4:]: v for k, v in t.items() if k.startswith("mlp.")}
            self.ff = FEED_FORWARDS[spec.mlp["kind"]](spec.mlp, width, mlp, device, f32)
        self.norm1 = _f32(t["norm1"].reshape(1), device)
        rows = list(self.mixer.in_rows) + [("rg1", t["rg1"])]
        self.rg1_b = _f32(t["rg1.b"], device)
        self.rg2_b = None
        if self.ff is not None:
            rows.append(("rg2", t["rg2"]))
            self.rg2_b = _f32(t["rg2.b"], device)
        self.col = {}
        off = 0
        parts = []
        for name, w in rows:
            self.col[name] = (off, w.shape[0])
            w = _pad8(w)
            parts.append(w)
            off += w.shape[0]
        if off % 64:  # whole 64-column tiles: the widest alignment any of the GEMMs asks for
            parts.append(torch.zeros(64 - off % 64, width, dtype=parts[0].dtype))
        self.proj = Proj(torch.cat(parts), device, f32)
        del self.mixer.in_rows

    def cols(self, P: torch.Tensor, name: str) -> torch.Tensor:
        a, n = self.col[name]
        return P[:, a: a + n]

    def nbytes(self) -> int:
        return self.proj.nbytes() + self.mixer.nbytes() + (self.ff.nbytes() if self.ff else 0)


class HybridModel:
    stateful = True  # recurrent state: no prefix reuse, no recompute from a cached prefix

    def __init__(self, arch: HybridArch, device, tp: TPGroup | None = None, quantization: str | None = None,
                 seed: int = 0, weights_path: str | None = None, max_model_len: int = 4096,
                 dtype: str = "bfloat16"):
        self.arch = arch
        self.device = torch.device(device)
        self.tp = tp or TPGroup()
        if self.tp.size > 1:
            raise ValueError("layered hybrid models run on one GPU per replica (tensor_parallel_size 1)")
        if (quantization or "none").lower() not in ("none", ""):
            raise ValueError(f"layered hybrid models have no quantized path (quantization={quantization!r})")
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype {dtype!r}: bfloat16 or float32")
        self.f32 = dtype == "float32"
        self.act_dtype = torch.float32 if self.f32 else torch.bfloat16
        self.max_model_len = max_model_len
        W = arch.hidden_size
        tensors = load_tensors(arch, weights_path) if weights_path else random_tensors(arch, seed)
        self.embed = tensors["embed"].to(self.device, self.act_dtype).contiguous()
        owned: dict[int, LayerWeights] = {}
        self.layers: list[LayerWeights] = []
        for i, spec in enumerate(arch.layers):
            j = arch.owner(i)
            if j not in owned:
                pre = f"l{j}."
                t = {k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}
                owned[j] = LayerWeights(arch.layers[j], W, arch.rms_eps, t, self.device, self.f32)
            if MIXERS[spec.kind] is not type(owned[j].mixer):
                raise ValueError(f"layer {i} shares weights with layer {j} of another mixer type")
            self.layers.append(owned[j])
        self._owned = owned
        self.final_norm = _f32(tensors["final.norm"].reshape(1), self.device)
        self.head = Proj(tensors["head"], self.device, self.f32)
        self.capture_layers: list | None = None  # set to [] to record the residual stream after every layer
        self.last_resid = None

    # ------------------------------------------------------------------ sizes
    def weight_bytes(self) -> int:
        return (self.embed.numel() * self.embed.element_size() + self.head.nbytes()
                + sum(L.nbytes() for L in self._owned.values()))

    def cache_bytes_per_block(self, block_size: int) -> int:
        """Bytes one cache page costs over all layers with a paged cache."""
        n = 0
        for L in self.layers:
            if L.mixer.cache == "paged":
                s = L.mixer.cache_shape(1, block_size, 1)
                n += math.prod(s) * torch.empty(0, dtype=L.mixer.cache_dtype()).element_size()
        return max(n, 1)

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int) -> list:
        """One tensor per layer: a paged cache [blocks, page, row] or a state [slots, ...] (zeroed:
        stale rows are always finite)."""
        return [torch.zeros(L.mixer.cache_shape(num_blocks, block_size, num_slots), dtype=L.mixer.cache_dtype(),
                            device=self.device) for L in self.layers]

    # ---------------------------------------------------------------- forward
    def forward(self, sv, caches, part_size: int = 0, return_hidden: bool = False) -> torch.Tensor:
        """One step. Returns fp32 logits [S, vocab] of the sample rows, or with ``return_hidden`` the
        fp32 residual stream [T, width] after the last layer."""
        T = sv.T
        W = self.arch.hidden_size
        dev, eps = self.device, self.arch.rms_eps
        x = torch.empty(T, W, dtype=torch.float32, device=dev)
        seq.embed_rows(sv.ids, self.embed, x, prev=sv.prev_tokens)
        h = torch.empty(T, W, dtype=self.act_dtype, device=dev)
        for li, L in enumerate(self.layers):
            seq.norm_rows(x, L.norm1, eps, h, scalar=True)
            P = L.proj(h)
            y1 = L.mixer.forward(h, P, L.cols, sv, caches[li])
            y2 = L.ff.forward(h) if L.ff is not None else None
            seq.gated_residual(x, y1, L.cols(P, "rg1"), L.rg1_b, y2, L.cols(P, "rg2") if y2 is not None else None,
                               L.rg2_b)
            if self.capture_layers is not None:
                self.capture_layers.append(x.clone())
        self.last_resid = x
        if return_hidden:
            return x
        V = self.arch.vocab_size
        if V % 4 == 0:
            return self.logits_of(x, sv.sample_idx)
        # the sampler reads rows of whole 16-B pieces: pad the row with -inf columns (never sampled)
        buf = torch.full((sv.sample_idx.numel(), (V + 3) // 4 * 4), float("-inf"), dtype=torch.float32, device=dev)
        self.logits_of(x, sv.sample_idx, out=buf[:, :V])
        return buf

    def logits_of(self, x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """fp32 logits [len(rows), vocab] of rows of the residual stream (final norm + head)."""
        hn = torch.empty(rows.numel(), x.shape[1], dtype=self.act_dtype, device=x.device)
        seq.norm_rows(x, self.final_norm, self.arch.rms_eps, hn, rows=rows, scalar=True)
        return self.head(hn, out_f32=True, out=out)[:, : self.arch.vocab_size]


# ------------------------------------------------------------------------------------------ weights
def tensor_shapes(arch: HybridArch) -> dict:
    """name -> shape of every tensor of a checkpoint of ``arch`` (weight-owning layers only)."""
    W = arch.hidden_size
    out = {"embed": (arch.vocab_size, W), "final.norm": (), "head": (arch.vocab_size, W)}
    for i in sorted({arch.owner(i) for i in range(arch.num_layers)}):
        out.update({f"l{i}.{k}": v for k, v in layer_shapes(arch.layers[i], W).items()})
    return out


def load_tensors(arch: HybridArch, path: str) -> dict:
    """Read ``model.safetensors`` (bf16 tensors, row-major [out, in]) of a layered hybrid checkpoint
    and check every tensor the architecture needs against its expected shape. Sizes the config does
    not carry (the decay low-rank width) come from the tensors."""
    from safetensors import safe_open
    root = Path(path)
    files = sorted(root.glob("*.safetensors")) if root.is_dir() else [root]
    if not files:
        raise FileNotFoundError(f"no *.safetensors under {root}")
    t = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as h:
            for k in h.keys():
                t[k] = h.get_tensor(k)
    for name, shape in tensor_shapes(arch).items():
        if name not in t:
            raise KeyError(f"checkpoint lacks tensor {name}")
        got = tuple(t[name].shape)
        if name.endswith("mix.w1"):
            ok = len(got) == 2 and got[1] == shape[1]
        elif name.endswith("mix.w2"):
            ok = len(got) == 2 and got[0] == shape[0] and got[1] == t[name[:-1] + "1"].shape[0]
        else:
            ok = got == tuple(shape) or (math.prod(got) == 1 and math.prod(shape) == 1)
        if not ok:
            raise ValueError(f"tensor {name}: shape {got}, expected {tuple(shape)}")
    return t


def random_tensors(arch: HybridArch, seed: int = 0) -> dict:
    """Seeded random bf16 weights (benchmarks / tests): matrices ~ N(0, 1 / fan_in), norm weights near 1,
    biases and corrections small, so activations stay O(1) through any depth."""
    g = torch.Generator().manual_seed(seed * 1000003 + 17)
    out = {}
    for name, shape in tensor_shapes(arch).items():
        leaf = name.split(".")[-1] if not name.endswith(".b") else "b"
        if len(shape) == 2:
            std = 0.5 if name == "embed" else 1.0 / math.sqrt(shape[1])
            w = torch.randn(shape, generator=g) * std
        elif leaf in ("norm", "norm1") or name == "final.norm":
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        else:
            w = 0.3 * torch.randn(shape, generator=g)
        out[name] = w.to(torch.bfloat16)
    return out


def save_checkpoint(arch: HybridArch, tensors: dict, path: str, config: dict) -> None:
    """Write ``config.json`` + ``model.safetensors`` of a layered hybrid model."""
    from safetensors.torch import save_file
    Path(path).mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(Path(path) / "model.safetensors"))
    (Path(path) / "config.json").write_text(json.dumps(config, indent=1))
