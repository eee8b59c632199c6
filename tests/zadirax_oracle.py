"""Plain, slow fp32 implementation of the Zadirax design, one function per mechanism, written from the
design's equations and sharing no code with ``vgate`` (tests compare the framework against it).

Notation: n tokens, width d, heads H. Linear maps are applied as ``x @ M.T`` for M stored [out, in].
Every function takes the whole sequence (positions 0..n-1) and recomputes everything.
"""
from __future__ import annotations

import math

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(torch.mean(x * x, dim=-1, keepdim=True) + eps)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def rotate_pairs(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [n, ..., m]: entries (2i, 2i+1), i < dims/2, turn by the angle p * base^(-2i/dims) at position p."""
    n = x.shape[0]
    out = x.clone()
    for p in range(n):
        for i in range(dims // 2):
            ang = torch.tensor(float(p), dtype=torch.float32) * (torch.tensor(base, dtype=torch.float32) ** (-2.0 * i / dims))
            c, s = torch.cos(ang), torch.sin(ang)
            a, b = x[p, ..., 2 * i], x[p, ..., 2 * i + 1]
            out[p, ..., 2 * i] = a * c - b * s
            out[p, ..., 2 * i + 1] = b * c + a * s
    return out


def latent_attention(m: dict, W: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """W: 'dq', 'dq.norm', 'uq', 'dkv', 'dkv.norm', 'uk', 'uv', 'g', 'o' (fp32)."""
    n = h.shape[0]
    H, D, R, V, KR = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (unit_rms(h @ W["dq"].T, eps) * W["dq.norm"]) @ W["uq"].T
    q = q.reshape(n, H, D + R)
    low = h @ W["dkv"].T
    c = unit_rms(low[:, :KR], eps) * W["dkv.norm"]
    shared = rotate_pairs(low[:, KR:], m["rot"]["base"], m["rot"]["dims"])
    q_rot = rotate_pairs(q[:, :, D:], m["rot"]["base"], m["rot"]["dims"])
    keys = (c @ W["uk"].T).reshape(n, H, D)
    vals = (c @ W["uv"].T).reshape(n, H, V)
    out = torch.zeros(n, H, V)
    for i in range(n):
        for hh in range(H):
            sc = torch.stack([(q[i, hh, :D] @ keys[j, hh] + q_rot[i, hh] @ shared[j]) * m["scale"] for j in range(i + 1)])
            p = torch.softmax(sc, 0)
            out[i, hh] = (p[:, None] * vals[: i + 1, hh]).sum(0)
    out = out.reshape(n, H * V) * sigmoid(h @ W["g"].T)
    return out @ W["o"].T


def general_delta(m: dict, W: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """W: 'r', 'k', 'v', 'g', 'a', 'a.b', 'w1', 'w2', 'w0', 'norm', 'o'."""
    n = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ W["r"].T).reshape(n, H, D)
    k = (h @ W["k"].T).reshape(n, H, D)
    v = (h @ W["v"].T).reshape(n, H, D)
    decay = torch.exp(-math.exp(-0.5) * sigmoid(torch.tanh(h @ W["w1"].T) @ W["w2"].T + W["w0"])).reshape(n, H, D)
    rate = sigmoid(h @ W["a"].T + W["a.b"]).reshape(n, H, D)
    o = torch.zeros(n, H, D)
    for hh in range(H):
        S = torch.zeros(D, D)  # rows: key channel, columns: value channel
        for t in range(n):
            u = k[t, hh] / torch.sqrt((k[t, hh] ** 2).sum() + 1e-6)
            S = torch.diag(decay[t, hh]) @ S - torch.outer(rate[t, hh] * u, u @ S) + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ r[t, hh]
    o = unit_rms(o, eps).reshape(n, H * D) * W["norm"] * sigmoid(h @ W["g"].T)
    return o @ W["o"].T


def dense_ff(W: dict, h: torch.Tensor) -> torch.Tensor:
    a = h @ W["gate"].T
    return ((a * sigmoid(a)) * (h @ W["up"].T)) @ W["down"].T


def moe_ff(f: dict, W: dict, h: torch.Tensor) -> torch.Tensor:
    E, top, lim = f["router"]["experts"], f["router"]["top"], f["expert"]["limit"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        s = sigmoid(W["router"] @ h[t])
        chosen = torch.argsort(s + W["correction"], descending=True, stable=True)[:top]
        total = s[chosen].sum() + 1e-20
        for e in chosen.tolist():
            g = torch.clamp(W[f"e{e}.gate"] @ h[t], max=lim)
            u = torch.clamp(W[f"e{e}.up"] @ h[t], -lim, lim)
            out[t] += (s[e] / total) * (W[f"e{e}.down"] @ (g * sigmoid(1.702 * g) * (u + 1.0)))
    return out


def sub(W: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def forward(cfg: dict, W: dict, tokens: list[int], layers_out: list | None = None) -> torch.Tensor:
    """fp32 logits [n, vocab] of one sequence from config.json's dict and the fp32 tensors by name."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    for i, L in enumerate(cfg["layers"]):
        own = f"l{L.get('weights_of', i) if L.get('weights_of') is not None else i}."
        h = unit_rms(x, eps) * W[own + "norm1"]
        mix = latent_attention if L["type"] == "latent_attention" else general_delta
        y = mix(L["mixer"], sub(W, own + "mix."), h, eps) * sigmoid(h @ W[own + "rg1"].T + W[own + "rg1.b"])
        if L.get("mlp"):
            f = L["mlp"]
            z = dense_ff(sub(W, own + "mlp."), h) if f["kind"] == "dense" else moe_ff(f, sub(W, own + "mlp."), h)
            y = y + z * sigmoid(h @ W[own + "rg2"].T + W[own + "rg2.b"])
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T
