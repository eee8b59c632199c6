"""Token mixers and feed-forwards of layered hybrid models, one class per mechanism.

A mixer reads the layer's normed input ``h`` through rows of the layer's fused input projection
(``in_rows``: every matrix that multiplies ``h`` is stacked into one GEMM by the model) and owns
the rest of its weights. Constants of a mechanism are constructor parameters read from the layer's
spec, so another design can reuse a mixer with other values.

* :class:`LatentAttention` — attention through a low-rank key/value latent with one rotated key part
  shared by all heads; only the latent and that part are cached (paged), the per-head up-projections
  are absorbed into the query and the output.
* :class:`GeneralDelta` — generalized delta rule with per-channel decay over an fp32 state matrix
  per head, kept in a state slot per sequence.
* :class:`DenseFF`, :class:`MoEFF` — gated feed-forward; sigmoid-routed mixture of clamped gated experts.
"""
from __future__ import annotations

import math
import os

import torch

from vgate import ops
from vgate.ops import seq

# bf16 matrices in the shape range the fragment-packed MFMA GEMMs are exercised on (N and K multiples
# of 64, K >= 512: the transformer families' projections) run there; the rest (and every fp32 matrix)
# through the row-major GEMM. "0" sends everything through the row-major one.
USE_PACKED = os.environ.get("VGATE_HYBRID_PACKED", "1") == "1"
PACKED_MIN_K = 512


class Proj:
    """y = x W^T for a [N, K] matrix, on whichever GEMM takes its shape and dtype."""

    def __init__(self, w: torch.Tensor, device, f32: bool, silu_pair: bool = False, allow_packed: bool = True):
        N, K = w.shape
        self.N, self.K, self.f32, self.silu_pair = N, K, f32, silu_pair
        dev = torch.device(device)
        n_ok = (N // 2) % 64 == 0 if silu_pair else N % 64 == 0
        self.packed = (USE_PACKED and allow_packed and not f32 and dev.type == "cuda" and n_ok and K % 64 == 0
                       and K >= PACKED_MIN_K)
        if self.packed:
            self.lin = ops.Linear(w.to(dev, torch.bfloat16), kind="silu" if silu_pair else "plain")
            self.w = None
        else:
            self.lin = None
            self.w = w.to(dev, torch.float32 if f32 else torch.bfloat16).contiguous()
        self.out_features = N // 2 if silu_pair else N

    def nbytes(self) -> int:
        return self.lin.nbytes() if self.packed else self.w.numel() * self.w.element_size()

    def __call__(self, x: torch.Tensor, out_f32: bool = False, act: int = 0, out: torch.Tensor | None = None) -> torch.Tensor:
        M = x.shape[0]
        if self.packed and act == 0:
            return ops.linear(x, self.lin, out=out, out_f32=out_f32)
        dt = torch.float32 if (out_f32 or self.f32) else torch.bfloat16
        if out is None:
            out = torch.empty(M, self.out_features, dtype=dt, device=x.device)
        if self.silu_pair:
            I = self.N // 2
            return seq.gemm(x, self.w[:I], out, w2=self.w[I:], act=seq.ACT_SILU_MUL)
        return seq.gemm(x, self.w, out, act=act)


def _f32(t: torch.Tensor, device) -> torch.Tensor:
    return t.to(device, torch.float32).contiguous()


def _pad8(w: torch.Tensor) -> torch.Tensor:
    """Zero rows up to a multiple of 8, so every segment of a fused projection starts 16-B aligned."""
    n = (-w.shape[0]) % 8
    return torch.cat([w, torch.zeros(n, w.shape[1], dtype=w.dtype)]) if n else w


# ------------------------------------------------------------------------------------------ mixers
class LatentAttention:
    kind = "latent_attention"
    cache = "paged"
    TENSORS = ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o")

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool):
        m = spec
        self.H, self.D, self.R, self.V = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
        self.KR, self.QR = int(m["kv_rank"]), int(m["q_rank"])
        self.scale = float(m["scale"])
        rot = m.get("rot") or {}
        dims = int(rot.get("dims", self.R))
        if dims > self.R or dims < 0:
            raise ValueError("latent_attention: rot.dims must be <= rot_dim")
        self.rot_dims = 2 * (dims // 2)  # entries in rotated pairs (an odd last one passes unchanged)
        self.eps = eps
        self.f32 = f32
        dev = torch.device(device)
        H, D, R, V, KR = self.H, self.D, self.R, self.V, self.KR
        self.inv_freq = seq.rope_inv_freq(dims, float(rot.get("base", 10000.0)), dev)  # base^(-2i / dims)
        self.in_rows = [("dq", tensors["dq"]), ("dkv", tensors["dkv"]), ("g", tensors["g"])]
        self.dq_norm, self.dkv_norm = _f32(tensors["dq.norm"], dev), _f32(tensors["dkv.norm"], dev)
        self.uq = Proj(tensors["uq"], dev, f32)
        dt = torch.float32 if f32 else torch.bfloat16
        # absorbed up-projections, one matrix per head: q' = q_h W_uk[h] ([KR, D] as the GEMM's W), out = ol W_uv[h]^T
        self.uk_t = tensors["uk"].view(H, D, KR).transpose(1, 2).contiguous().to(dev, dt)
        self.uv = tensors["uv"].view(H, V, KR).contiguous().to(dev, dt)
        self.o = Proj(tensors["o"], dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        H, D, R, V = spec["heads"], spec["dim"], spec["rot_dim"], spec["vdim"]
        KR, QR = spec["kv_rank"], spec["q_rank"]
        return {"dq": (QR, width), "dq.norm": (QR,), "uq": (H * (D + R), QR), "dkv": (KR + R, width),
                "dkv.norm": (KR,), "uk": (H * D, KR), "uv": (H * V, KR), "g": (H * V, width), "o": (width, H * V)}

    def cache_shape(self, num_blocks: int, block_size: int, num_slots: int) -> tuple:
        """One flat buffer per layer: rows [blocks, page, kv_rank + rot_dim], then (bf16) the transposed copy of
        the latent part [blocks, kv_rank, page] that the MFMA attention kernel reads."""
        self._page = block_size
        return (num_blocks * block_size * (self.KR + self.R + (0 if self.f32 else self.KR)),)

    def _views(self, cache: torch.Tensor):
        E, block_size = self.KR + self.R, getattr(self, "_page", 16)
        per = block_size * (E + (0 if self.f32 else self.KR))
        nb = cache.numel() // per
        rows = cache[: nb * block_size * E].view(nb, block_size, E)
        tr = None if self.f32 else cache[nb * block_size * E:].view(nb, self.KR, block_size)
        return rows, tr

    def cache_dtype(self):
        return torch.float32 if self.f32 else torch.bfloat16

    def nbytes(self) -> int:
        return self.uq.nbytes() + self.o.nbytes() + 2 * self.uk_t.numel() * self.uk_t.element_size()

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        H, D, R, V, KR = self.H, self.D, self.R, self.V, self.KR
        E = KR + R
        dt, dev = h.dtype, h.device
        cq = torch.empty(T, self.QR, dtype=dt, device=dev)
        seq.norm_rows(cols(P, "dq"), self.dq_norm, self.eps, cq)
        q = self.uq(cq)
        cache, cache_t = self._views(cache)
        seq.latent_write(cols(P, "dkv"), self.dkv_norm, self.eps, sv.positions, sv.slots, self.inv_freq,
                         self.rot_dims, cache, KR, cache_t=cache_t)
        qa = torch.empty(T, H, E, dtype=dt, device=dev)
        seq.gemm(q.view(T, H, D + R)[:, :, :D].permute(1, 0, 2), self.uk_t, qa[:, :, :KR].permute(1, 0, 2))
        seq.latent_qrope(q, sv.positions, self.inv_freq, self.rot_dims, qa, H, D, KR, R)
        ol = torch.empty(T, H, KR, dtype=dt, device=dev)
        seq.latent_attn(qa, cache, sv.block_tables, sv.context_lens, sv.query_start, ol, self.scale, H, KR, R,
                        num_seqs=sv.num_seqs or None, cache_t=cache_t)
        og = torch.empty(T, H, V, dtype=dt, device=dev)
        gate = cols(P, "g").unflatten(1, (H, V)).permute(1, 0, 2)
        seq.gemm(ol.permute(1, 0, 2), self.uv, og.permute(1, 0, 2), gate=gate)
        return self.o(og.view(T, H * V))


class GeneralDelta:
    kind = "general_delta"
    cache = "state"
    TENSORS = ("r", "k", "v", "g", "a", "a.b", "w1", "w2", "w0", "norm", "o")
    DECAY_C = math.exp(-0.5)   # w = exp(-DECAY_C * sigmoid(.))
    UNIT_EPS = 1e-6            # u = k / sqrt(sum(k^2) + UNIT_EPS)

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool,
                 decay_c: float | None = None, unit_eps: float | None = None):
        self.H, self.D = int(spec["heads"]), int(spec["dim"])
        if self.D > 128:
            raise ValueError("general_delta: the recurrence kernel keeps a state column in registers: head size <= 128")
        self.eps, self.f32 = eps, f32
        self.decay_c = self.DECAY_C if decay_c is None else decay_c
        self.unit_eps = self.UNIT_EPS if unit_eps is None else unit_eps
        dev = torch.device(device)
        self.in_rows = [(n, tensors[n]) for n in ("r", "k", "v", "g", "a")]
        self.w1 = Proj(tensors["w1"], dev, f32, allow_packed=False)  # tanh in its epilogue
        self.w2 = Proj(tensors["w2"], dev, f32)
        self.w0, self.ab, self.nw = _f32(tensors["w0"], dev), _f32(tensors["a.b"], dev), _f32(tensors["norm"], dev)
        self.o = Proj(tensors["o"], dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        n = spec["heads"] * spec["dim"]
        decay_rank = int(spec.get("decay_rank", 16))  # checkpoints: the shape of w1 gives it
        return {"r": (n, width), "k": (n, width), "v": (n, width), "g": (n, width), "a": (n, width), "a.b": (n,),
                "w1": (decay_rank, width), "w2": (n, decay_rank), "w0": (n,), "norm": (n,), "o": (width, n)}

    def cache_shape(self, num_blocks: int, block_size: int, num_slots: int) -> tuple:
        return (num_slots, self.H, self.D, self.D)

    def cache_dtype(self):
        return torch.float32

    def nbytes(self) -> int:
        return self.w1.nbytes() + self.w2.nbytes() + self.o.nbytes()

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        wl = self.w2(self.w1(h, act=seq.ACT_TANH))
        out = torch.empty(T, self.H * self.D, dtype=h.dtype, device=h.device)
        seq.delta_rule(cols(P, "r"), cols(P, "k"), cols(P, "v"), cols(P, "g"), cols(P, "a"), wl, self.w0, self.ab,
                       self.nw, cache, sv.state_slots, sv.context_lens, sv.query_start, out, self.decay_c,
                       self.unit_eps, self.eps, num_seqs=sv.num_seqs or None)
        return self.o(out)


MIXERS = {c.kind: c for c in (LatentAttention, GeneralDelta)}


# ------------------------------------------------------------------------------------ feed-forwards
class DenseFF:
    """down(silu(gate h) * (up h))."""

    def __init__(self, spec: dict, width: int, tensors: dict, device, f32: bool):
        self.gate_up = Proj(torch.cat([tensors["gate"], tensors["up"]]), device, f32, silu_pair=True)
        self.down = Proj(tensors["down"], device, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        return {"gate": (spec["ff"], width), "up": (spec["ff"], width), "down": (width, spec["ff"])}

    def nbytes(self) -> int:
        return self.gate_up.nbytes() + self.down.nbytes()

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(self.gate_up(h))


class MoEFF:
    """Sigmoid-routed experts: the ``top`` largest of sigmoid(z) + correction are chosen, weighted by
    their uncorrected scores over the sum. Expert: g = min(gate h, L), u = clamp(up h, -L, L),
    down(g * sigmoid(alpha g) * (u + 1))."""
    ALPHA = 1.702
    SUM_EPS = 1e-20

    def __init__(self, spec: dict, width: int, tensors: dict, device, f32: bool):
        self.E, self.top = int(spec["router"]["experts"]), int(spec["router"]["top"])
        self.ff, self.limit = int(spec["expert"]["ff"]), float(spec["expert"]["limit"])
        dev = torch.device(device)
        dt = torch.float32 if f32 else torch.bfloat16
        self.f32 = f32
        self.router = Proj(tensors["router"], dev, f32, allow_packed=False)  # fp32 logits, N = experts
        self.corr = _f32(tensors["correction"], dev)
        st = lambda n: torch.stack([tensors[f"e{e}.{n}"] for e in range(self.E)]).to(dev, dt).contiguous()  # noqa: E731
        self.gate, self.up, self.down = st("gate"), st("up"), st("down")

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        E, ff = spec["router"]["experts"], spec["expert"]["ff"]
        out = {"router": (E, width), "correction": (E,)}
        for e in range(E):
            out.update({f"e{e}.gate": (ff, width), f"e{e}.up": (ff, width), f"e{e}.down": (width, ff)})
        return out

    def nbytes(self) -> int:
        return self.router.nbytes() + 3 * self.gate.numel() * self.gate.element_size()

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        T, W = h.shape
        dev, dt = h.device, h.dtype
        z = self.router(h, out_f32=True)
        idx = torch.empty(T, self.top, dtype=torch.int32, device=dev)
        wts = torch.empty(T, self.top, dtype=torch.float32, device=dev)
        seq.moe_route(z, self.corr, self.top, self.SUM_EPS, idx, wts)
        rows = torch.empty(T * self.top, dtype=torch.int32, device=dev)
        pos = torch.empty(T * self.top, dtype=torch.int32, device=dev)
        off = torch.empty(self.E + 1, dtype=torch.int32, device=dev)
        seq.moe_sort(idx, self.E, rows, pos, off)
        a1 = torch.empty(T * self.top, self.ff, dtype=dt, device=dev)
        seq.gemm(h, self.gate, a1, w2=self.up, a_rows=rows, group_off=off, act=seq.ACT_CLAMPED_GLU, limit=self.limit,
                 alpha=self.ALPHA)
        y = torch.empty(T * self.top, W, dtype=dt, device=dev)
        seq.gemm(a1, self.down, y, group_off=off)
        out = torch.empty(T, W, dtype=dt, device=dev)
        seq.moe_combine(y, pos, wts, out)
        return out


FEED_FORWARDS = {"dense": DenseFF, "moe": MoEFF}


def layer_shapes(spec, width: int) -> dict:
    """name -> shape of every tensor of a layer that owns its weights (suffixes after 'l<i>.')."""
    out = {"norm1": ()}
    out.update({"mix." + k: v for k, v in MIXERS[spec.kind].shapes(spec.mixer, width).items()})
    out.update({"rg1": (width, width), "rg1.b": (width,)})
    if spec.mlp:
        out.update({"mlp." + k: v for k, v in FEED_FORWARDS[spec.mlp["kind"]].shapes(spec.mlp, width).items()})
        out.update({"rg2": (width, width), "rg2.b": (width,)})
    return out


def layer_params(spec, width: int) -> int:
    return sum(math.prod(s) for s in layer_shapes(spec, width).values())
