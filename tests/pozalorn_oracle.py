"""Plain, slow implementation of the Pozalorn design, one function per mechanism, written from the
equations alone (it shares no code with ``vgate``). Everything runs in one floating-point type
(fp32 by default, fp64 to measure rounding), token by token where a mechanism is recurrent and key
by key where it attends.

Weights: a dict name -> tensor as in a checkpoint (``l<i>.mix.q`` ...), matrices [out, in].
"""
from __future__ import annotations

import math

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------------ rotation
def frequencies(n_dims: int, base: float, scaling: dict | None, dtype) -> torch.Tensor:
    """f_i = base^(-2i / n_dims); with ``scaling`` long wavelengths are slowed down by ``factor`` and a
    band between original / low and original / high is blended."""
    out = []
    for i in range(n_dims // 2):
        f = float(base) ** (-2.0 * i / n_dims)
        if scaling:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave < orig / hi:
                pass
            elif wave > orig / lo:
                f = f / fac
            else:
                s = (orig / wave - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=dtype)


def turn_pairs(x: torch.Tensor, pos: float, freqs: torch.Tensor, n_dims: int) -> torch.Tensor:
    """Entries (2i, 2i + 1), i < n_dims / 2, of a vector turned by pos * freqs[i]; the rest unchanged."""
    y = x.clone()
    for i in range(n_dims // 2):
        a = torch.tensor(pos, dtype=x.dtype) * freqs[i]
        c, s = torch.cos(a), torch.sin(a)
        u, v = x[2 * i], x[2 * i + 1]
        y[2 * i] = u * c - v * s
        y[2 * i + 1] = v * c + u * s
    return y


# -------------------------------------------------------------------------------------------- mixers
def recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor, S: torch.Tensor | None = None):
    """One head: S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t. q, k, a [T, D]; v [T, V]. Returns (o, S)."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=q.dtype) if S is None else S.clone()
    o = []
    for t in range(T):
        S = a[t][:, None] * S + k[t][:, None] * v[t][None, :]
        o.append(S.t() @ q[t])
    return torch.stack(o), S


def attend(q: torch.Tensor, keys: list, vals: list, t: int, size: int, pool: int, scale: float, sink) -> torch.Tensor:
    """Position t's attention output [H, V]: q [H, D]; keys[j] [G, D] and vals[j] [G, V] of positions 0 .. t."""
    H, G = q.shape[0], keys[0].shape[0]
    ks, vs = [], []
    if pool:
        b = 0
        while b * pool + pool - 1 <= t - size:
            ks.append(torch.stack(keys[b * pool: b * pool + pool]).mean(0))
            vs.append(torch.stack(vals[b * pool: b * pool + pool]).mean(0))
            b += 1
    lo = max(0, t - size + 1)
    K, V = torch.stack(ks + keys[lo: t + 1]), torch.stack(vs + vals[lo: t + 1])   # [n, G, D], [n, G, Dv]
    o = torch.zeros(H, V.shape[-1], dtype=q.dtype)
    for hd in range(H):
        g = hd // (H // G)
        sc = (K[:, g] @ q[hd]) * scale
        mx = sc.max() if sink is None else torch.maximum(sc.max(), sink[hd])
        e = torch.exp(sc - mx)
        den = e.sum() + (torch.exp(sink[hd] - mx) if sink is not None else 0.0)
        o[hd] = (e / den) @ V[:, g]
    return o


def gated_linear_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head; alpha = sigmoid(z)^(1 / tau)."""
    H, D, Dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    T = h.shape[0]
    q = (h @ w["q"].t()).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].t()).view(T, H, D)
    v = (h @ w["v"].t()).view(T, H, Dv)
    z = ((h @ w["a1"].t()) @ w["a2"].t() + w["a2.b"]).view(T, H, D)
    alpha = torch.sigmoid(z) ** (1.0 / tau)
    o = torch.stack([recurrence(q[:, i], k[:, i], v[:, i], alpha[:, i])[0] for i in range(H)], 1)   # [T, H, Dv]
    o = rms_unit(o, eps) * w["norm"]                # per head, one weight vector for all heads
    return (o.reshape(T, -1) * silu(h @ w["g"].t())) @ w["o"].t()


def lightning_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """S_t = decay_h S_(t-1) + k_t v_t^T with silu on q, k, v; the heads are normed together."""
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q, k, v = silu(h @ w["q"].t()).view(T, H, D), silu(h @ w["k"].t()).view(T, H, D), silu(h @ w["v"].t()).view(T, H, Dv)
    o = torch.stack([recurrence(q[:, i], k[:, i], v[:, i], torch.full((T, D), float(m["decay"][i]), dtype=h.dtype))[0]
                     for i in range(H)], 1)
    o = rms_unit(o.reshape(T, -1), eps) * w["norm"]
    return (o * torch.sigmoid(h @ w["g"].t())) @ w["o"].t()


def window_attention(h: torch.Tensor, w: dict, m: dict, eps: float, norm_over: str, turn_values: bool,
                     out_bias: bool) -> torch.Tensor:
    """Grouped-query attention over a sliding window; optionally one mean key / value per block of
    ``mask.pool`` tokens that lies wholly before the window, optionally a sink in the denominator,
    optionally values turned by their position (and the output turned back by the query's)."""
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot, mask = m["rot"], m["mask"]
    size, pool = int(mask["size"]), int(mask.get("pool") or 0)
    fr = frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"), h.dtype)
    fv = frequencies(Dv, float(rot["base"]), None, h.dtype)
    sink = w.get("sink")
    T = h.shape[0]
    keys, vals = [], []
    out = []
    for t in range(T):
        x = h[t]
        q = w["q"] @ x + w["q.b"]
        k = w["k"] @ x + w["k.b"]
        v = (w["v"] @ x + w["v.b"]).view(G, Dv)
        if norm_over == "all":      # one norm over the whole projection
            q = (rms_unit(q, eps) * w["q.norm"]).view(H, D)
            k = (rms_unit(k, eps) * w["k.norm"]).view(G, D)
        else:                       # per head, one weight vector for all heads
            q = rms_unit(q.view(H, D), eps) * w["q.norm"]
            k = rms_unit(k.view(G, D), eps) * w["k.norm"]
        q = torch.stack([turn_pairs(q[i], t, fr, int(rot["dims"])) for i in range(H)])
        k = torch.stack([turn_pairs(k[i], t, fr, int(rot["dims"])) for i in range(G)])
        if turn_values:
            v = torch.stack([turn_pairs(v[i], t, fv, Dv) for i in range(G)])
        keys.append(k)
        vals.append(v)
        o = attend(q, keys, vals, t, size, pool, float(m["scale"]), sink)
        if turn_values:
            o = torch.stack([turn_pairs(o[i], -t, fv, Dv) for i in range(H)])
        y = w["o"] @ o.reshape(-1)
        out.append(y + w["o.b"] if out_bias else y)
    return torch.stack(out)


def sub(w: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def mixer(kind: str, h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    if kind == "gla":
        return gated_linear_attention(h, w, m, eps)
    if kind == "attention":
        return window_attention(h, w, m, eps, norm_over="all", turn_values=True, out_bias=False)
    if kind == "parallel":
        left = window_attention(h, sub(w, "left."), m["left"], eps, norm_over="head", turn_values=False, out_bias=True)
        right = lightning_attention(h, sub(w, "right."), m["right"], eps)
        return float(m["left_scale"]) * left + float(m["right_scale"]) * right
    raise ValueError(kind)


def dense_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].t()) * (h @ w["up"].t())) @ w["down"].t()


# --------------------------------------------------------------------------------------------- model
def forward(cfg: dict, W: dict, tokens: list, layers_out: list | None = None, dtype=torch.float32) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence. ``layers_out`` receives the stream after every layer
    (after the depth average)."""
    W = {k: v.to(dtype) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.tensor(tokens)]
    hist = [x]
    for i, L in enumerate(cfg["layers"]):
        w = sub(W, f"l{i}.")
        x = x + rms_unit(mixer(L["type"], x, sub(w, "mix."), L["mixer"], eps), eps) * w["norm1"]
        if L.get("mlp"):
            x = x + rms_unit(dense_ff(x, sub(w, "mlp.")), eps) * w["norm2"]
        hist.append(x)
        x = sum(w["dwa"][j] * hist[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x)
    return (rms_unit(x, eps) * W["final.norm"]) @ W["head"].t()
