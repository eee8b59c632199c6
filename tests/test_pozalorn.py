"""Pozalorn (post-norm layers with depth averaging; window attention with pooled blocks, sinks and
rotated values; gated linear attention; lightning attention beside sink attention) in the engine,
against the plain implementation of tests/pozalorn_oracle.py.

Small configurations with random weights are written to a temporary folder (config.json +
model.safetensors) and run through ``LLMEngine.replay_step`` / ``add_request`` on the CPU device
(unfused torch forms of the ops) and, marked ``gpu``, on the HIP kernels, in fp32 and bf16.
"""
from __future__ import annotations

import json
import math

import pytest
import torch

import pozalorn_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


# ------------------------------------------------------------------------------------ configurations
def _rot(base, dims, factor, orig, low=1.0, high=4.0):
    return {"base": base, "dims": dims, "scaling": {"factor": factor, "low": low, "high": high, "original": orig}}


def _gla(H, D, V, tau, mlp):
    return {"type": "gla", "mixer": {"heads": H, "dim": D, "vdim": V, "tau": tau}, "mlp": mlp}


def _attn(H, G, D, V, size, pool, rot, mlp, scale=None):
    return {"type": "attention", "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "mask": {"size": size, "pool": pool},
                                           "rot": rot, "scale": scale or 1.0 / math.sqrt(D)}, "mlp": mlp}


def _par(H, G, D, V, size, rot, RH, RD, RV, decay, ls, rs, mlp):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "mask": {"size": size}, "rot": rot,
                               "scale": 1.3 / math.sqrt(D)},
                      "right": {"heads": RH, "dim": RD, "vdim": RV, "decay": decay}, "left_scale": ls, "right_scale": rs}}


def _ff(n):
    return {"kind": "dense", "ff": n}


def config_a():
    """Unequal everything: key size != value size, fewer rotated dims than the head, a pool that divides
    neither the page nor the window, a layer without feed-forward, a vocabulary that is not a multiple of 4."""
    return {"architecture": "Pozalorn", "width": 40, "vocab": 50, "norm": {"eps": 1e-5}, "layers": [
        _par(4, 2, 12, 10, 7, _rot(1000.0, 8, 3.0, 16), 3, 6, 10, [0.5, 0.9, 0.99], 0.7, 1.3, _ff(24)),
        _gla(2, 12, 6, 4.0, None),
        _attn(6, 3, 8, 6, 9, 3, _rot(100.0, 6, 2.0, 8, 1.0, 2.0), _ff(16)),
        _gla(3, 5, 9, 7.0, _ff(12))]}


def config_b():
    """Values that are 1 or equal: one head everywhere, window 1 beside pool 1 (everything earlier is seen
    through pooled rows), a window of 2 with a sink, tau 1, no scaling band (low = high would divide by zero: far apart)."""
    return {"architecture": "Pozalorn", "width": 24, "vocab": 32, "norm": {"eps": 1e-6}, "layers": [
        _attn(1, 1, 4, 4, 1, 1, _rot(10.0, 4, 1.0, 4), _ff(8)),
        _par(1, 1, 6, 6, 2, _rot(50.0, 6, 8.0, 32), 1, 4, 4, [0.8], 1.0, 1.0, None),
        _gla(1, 5, 5, 1.0, _ff(8))]}


def config_c():
    """Page-scale geometry: a pool larger than a page, one equal to half a page, windows that end inside pages."""
    return {"architecture": "Pozalorn", "width": 64, "vocab": 96, "norm": {"eps": 1e-6}, "layers": [
        _attn(4, 2, 16, 32, 37, 24, _rot(10000.0, 16, 4.0, 64), _ff(48)),
        _gla(2, 16, 24, 8.0, _ff(48)),
        _attn(2, 2, 32, 16, 20, 8, _rot(500.0, 24, 2.0, 32), None),
        _par(4, 1, 16, 16, 19, _rot(2000.0, 16, 2.0, 16), 2, 32, 16, [0.95, 0.7], 1.1, 0.6, _ff(32))]}


def config_d():
    """Sizes in the range the fragment-packed MFMA GEMMs take (width 512, projections in multiples of 64)."""
    return {"architecture": "Pozalorn", "width": 512, "vocab": 640, "norm": {"eps": 1e-6}, "layers": [
        _gla(4, 64, 64, 16.0, _ff(512)),
        _attn(8, 2, 64, 64, 24, 8, _rot(10000.0, 64, 4.0, 32), _ff(512)),
        _par(4, 2, 64, 64, 12, _rot(10000.0, 32, 2.0, 32), 2, 64, 128, [0.9, 0.99], 1.2, 0.8, _ff(512))]}


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d}


def make_tensors(cfg: dict, seed: int, gate_rank: int = 3) -> dict:
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.5):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    def window(p, m, per_head, sink, out_bias):
        H, G, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t = {p + "q": mat(H * D, W, 2.0), p + "k": mat(G * D, W, 2.0), p + "v": mat(G * Vd, W), p + "o": mat(W, H * Vd),
             p + "q.b": vec(H * D), p + "k.b": vec(G * D), p + "v.b": vec(G * Vd),
             p + "q.norm": vec(D if per_head else H * D, 1.0, 0.3), p + "k.norm": vec(D if per_head else G * D, 1.0, 0.3)}
        if sink:
            t[p + "sink"] = vec(H, 0.5, 1.0)
        if out_bias:
            t[p + "o.b"] = vec(W)
        return t

    t = {"embed": torch.randn(V, W, generator=g).to(torch.bfloat16), "head": mat(V, W), "final.norm": vec(W, 1.1, 0.2)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = vec(W, 0.8, 0.2)
        t[p + "dwa"] = vec(i + 2, 0.0, 0.3)
        t[p + "dwa"][-1] += 1.0
        if L["type"] == "gla":
            H, D, Vd = m["heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": mat(H * D, W, 2.0), p + "mix.k": mat(H * D, W, 2.0), p + "mix.v": mat(H * Vd, W),
                      p + "mix.g": mat(H * Vd, W), p + "mix.o": mat(W, H * Vd), p + "mix.norm": vec(Vd, 1.0, 0.3),
                      p + "mix.a1": mat(gate_rank, W), p + "mix.a2": mat(H * D, gate_rank, 3.0), p + "mix.a2.b": vec(H * D, 2.0, 1.0)})
        elif L["type"] == "attention":
            t.update(window(p + "mix.", m, per_head=False, sink=False, out_bias=False))
        else:
            t.update(window(p + "mix.left.", m["left"], per_head=True, sink=True, out_bias=True))
            r = m["right"]
            H, D, Vd = r["heads"], r["dim"], r["vdim"]
            q = p + "mix.right."
            t.update({q + "q": mat(H * D, W, 2.0), q + "k": mat(H * D, W, 2.0), q + "v": mat(H * Vd, W), q + "g": mat(H * Vd, W),
                      q + "o": mat(W, H * Vd), q + "norm": vec(H * Vd, 1.0, 0.3)})
        if L.get("mlp"):
            f = L["mlp"]["ff"]
            t.update({p + "norm2": vec(W, 0.8, 0.2), p + "mlp.gate": mat(f, W, 2.0), p + "mlp.up": mat(f, W), p + "mlp.down": mat(W, f)})
    return t


_MODELS: dict = {}


def model_dir(tmp_path_factory, name: str):
    """(folder, config dict, fp32 tensors) of a named test model, written once per session."""
    if name not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]()
        t = make_tensors(cfg, seed={"a": 3, "b": 5, "c": 7, "d": 9}[name], gate_rank=3 if name != "c" else 5)
        d = tmp_path_factory.mktemp("pozalorn_" + name)
        save_file({k: v.contiguous() for k, v in t.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[name] = (str(d), cfg, {k: v.float() for k, v in t.items()})
    return _MODELS[name]


_ORACLE: dict = {}


def oracle_logits(name, cfg, W, tokens):
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = oracle.forward(cfg, W, list(tokens))
    return _ORACLE[key]


def engine(path, device, dtype, pages=16, seqs=4, **kw):
    from vgate.runtime.engine import EngineConfig, LLMEngine
    cfg = dict(model=path, dtype=dtype, device=device, max_model_len=pages * 16, max_num_seqs=seqs,
               max_num_batched_tokens=pages * 16, num_kv_blocks=pages, enable_prefix_caching=False, enforce_eager=True,
               warmup=False, prefill_autotune=False, async_scheduling=False)
    cfg.update(kw)
    return LLMEngine(EngineConfig(**cfg))


def rel(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.float().cpu(), b.float().cpu()
    return float((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt())


def tol(dtype: str) -> float:
    return 3e-4 if dtype == "float32" else 6e-2


def tokens_of(cfg, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay_all(eng, rid, toks, cuts):
    """Run one request in portions of the given sizes (then one token at a time); logits at every place."""
    out, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - at)
        lg = eng.replay_step([(rid, toks[at: at + n], list(range(n)))], [rid] if at + n == len(toks) else [])
        out.append(lg.float().cpu())
        at += n
    return torch.cat(out)


# -------------------------------------------------------------------------------------------- engine
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt_matches_oracle(tmp_path_factory, device, dtype, name):
    path, cfg, W = model_dir(tmp_path_factory, name)
    toks = tokens_of(cfg, 90 if name == "c" else 37, seed=1)
    eng = engine(path, device, dtype)
    lg = replay_all(eng, "w", toks, [len(toks)])
    assert rel(lg, oracle_logits(name, cfg, W, toks)) < tol(dtype)
    one = replay_all(eng, "one", toks[:1], [1])  # a sequence of one token (first position only)
    assert rel(one, oracle_logits(name, cfg, W, toks)[:1]) < tol(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_oracle(tmp_path_factory, device):
    path, cfg, W = model_dir(tmp_path_factory, "a")
    toks = tokens_of(cfg, 23, seed=2)
    eng = engine(path, device, "float32")
    eng.model.capture_layers = []
    replay_all(eng, "l", toks, [len(toks)])
    want: list = []
    oracle.forward(cfg, W, toks, want)
    assert len(eng.model.capture_layers) == len(want) == len(cfg["layers"])
    for i, (got, w) in enumerate(zip(eng.model.capture_layers, want)):
        assert rel(got[: len(toks)], w) < 1e-4, f"stream handed on by layer {i}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[1], [30], [2, 2, 2, 3, 5, 7, 16, 17], [15, 1, 16, 2, 14], [47, 2]])
def test_portions_and_decoding_match_whole(tmp_path_factory, device, dtype, cuts):
    """Prefill against token-by-token decoding and portions of several sizes down to two tokens (cuts
    inside pages, windows and pooled blocks and at their borders); the tail decodes one token at a time
    until the windows have passed over decoded tokens."""
    path, cfg, W = model_dir(tmp_path_factory, "c")
    toks = tokens_of(cfg, 100, seed=3)
    eng = engine(path, device, dtype)
    whole = replay_all(eng, "whole", toks, [len(toks)])
    cut = replay_all(eng, "cut", toks, cuts)
    assert rel(cut, whole) < (2e-5 if dtype == "float32" else 3e-2)
    assert rel(cut, oracle_logits("c", cfg, W, toks)) < tol(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "c"])
def test_mixed_batches_and_reuse(tmp_path_factory, device, dtype, name):
    """Unequal requests in one batch (portions beside single tokens) against each alone, with a pool
    so small that pages and state slots are freed and taken again by later requests."""
    path, cfg, W = model_dir(tmp_path_factory, name)
    reqs = {f"q{i}": tokens_of(cfg, n, seed=10 + i) for i, n in enumerate([41, 5, 23, 1, 30, 17, 9, 48])}
    eng = engine(path, device, dtype, pages=8, seqs=3)  # 128 tokens, 3 slots: 8 requests must reuse both
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    order = list(reqs)
    live, step = [], 0
    plan = [7, 1, 16, 2, 1, 9, 3]
    while order or live:
        while order and len(live) < 3 and sum((len(reqs[k]) + 15) // 16 for k in live + [order[0]]) <= 8:
            live.append(order.pop(0))
        entries, end = [], []
        for j, k in enumerate(live):
            n = min(plan[(step + j) % len(plan)], len(reqs[k]) - at[k])
            if (step + j) % 5 == 4 and len(live) > 1:
                continue  # a request may sit a step out
            entries.append((k, reqs[k][at[k]: at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        step += 1
        if not entries:
            continue
        lg = eng.replay_step(entries, end).float().cpu()
        o = 0
        for k, t, w in entries:
            got[k].append(lg[o: o + len(w)])
            o += len(w)
        live = [k for k in live if k not in end]
    assert eng.kvm.num_free() == 8 and eng.kvm.free_state_slots() == 3
    for k, toks in reqs.items():
        assert rel(torch.cat(got[k]), oracle_logits(name, cfg, W, toks)) < tol(dtype), k


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(tmp_path_factory, device):
    """add_request -> scheduler (chunked prefill, continuous batching) -> sampler: every generated token
    is the oracle's arg-max (or within rounding of it) given the tokens before it."""
    from vgate.runtime.sampling_params import SamplingParams
    path, cfg, W = model_dir(tmp_path_factory, "a")
    eng = engine(path, device, "float32", pages=24, seqs=3, max_num_batched_tokens=24, enforce_eager=False)
    prompts = {"g0": tokens_of(cfg, 29, seed=31), "g1": tokens_of(cfg, 3, seed=32), "g2": tokens_of(cfg, 40, seed=33),
               "g3": tokens_of(cfg, 11, seed=34)}
    done = {}
    for rid, p in prompts.items():
        eng.add_request(rid, prompt_ids=p, params=SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True),
                        callback=lambda kind, seq, payload: done.__setitem__(seq.request_id, seq))
    eng.run_until_idle()
    assert set(done) == set(prompts)
    for rid, p in prompts.items():
        out = done[rid].output_ids
        assert len(out) == 12
        ref = oracle_logits("a", cfg, W, p + out[:-1])
        for i, tok in enumerate(out):
            row = ref[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (rid, i, tok, int(row.argmax()))
    assert eng.kvm.free_state_slots() == 3


@pytest.mark.gpu
def test_generation_replays_graphs(tmp_path_factory):
    """The second run of the same requests replays the hipGraphs captured after the first and samples
    the same tokens (bf16, the serving dtype)."""
    from vgate.runtime.sampling_params import SamplingParams
    path, cfg, W = model_dir(tmp_path_factory, "c")
    eng = engine(path, "cuda", "bfloat16", pages=32, seqs=4, enforce_eager=False)
    outs = []
    for rnd in range(2):
        done = {}
        for i in range(3):
            eng.add_request(f"r{rnd}_{i}", prompt_ids=tokens_of(cfg, 9 + 17 * i, seed=40 + i),
                            params=SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True),
                            callback=lambda kind, seq, payload: done.__setitem__(seq.request_id[3:], seq.output_ids))
        hits = eng.runner.graph_hits
        eng.run_until_idle()
        outs.append(done)
    assert eng.runner.graph_hits > hits
    assert outs[0] == outs[1]


@pytest.mark.gpu
def test_packed_gemm_path_matches_row_major_and_oracle(tmp_path_factory, monkeypatch):
    """bf16 at sizes whose projections run on the fragment-packed MFMA GEMMs (fused input projection with
    its bias, output projections with fp32 results): same logits as with every matrix on the row-major
    GEMM, and the oracle's; prompt portions and decoded tokens."""
    from vgate.models import mixers
    path, cfg, W = model_dir(tmp_path_factory, "d")
    toks = tokens_of(cfg, 45, seed=5)
    got = {}
    for packed in (True, False):
        monkeypatch.setattr(mixers, "USE_PACKED", packed)
        eng = engine(path, "cuda", "bfloat16")
        assert eng.model.layers[1].proj.packed == packed and eng.model.head.packed == packed
        got[packed] = replay_all(eng, "p", toks, [30, 2, 9])
        del eng
    assert rel(got[True], got[False]) < 3e-2
    assert rel(got[True], oracle_logits("d", cfg, W, toks)) < 0.2
    eng = engine(path, "cuda", "float32")
    assert rel(replay_all(eng, "f", toks, [30, 2, 9]), oracle_logits("d", cfg, W, toks)) < tol("float32")


def test_registry_and_config(tmp_path_factory):
    from vgate.models.config import HybridArch, resolve_arch
    from vgate.models.hybrid import tensor_shapes
    path, cfg, W = model_dir(tmp_path_factory, "a")
    a = resolve_arch(path)
    assert isinstance(a, HybridArch) and a.family == "pozalorn" and a.arrangement == "post_norm" and a.depth_average
    assert [L.kind for L in a.layers] == ["parallel", "linear_attention", "window_attention", "linear_attention"]
    assert a.layers[2].mixer["pool"] == 3 and a.layers[2].mixer["qk_norm"] == "all" and a.layers[2].mixer["rotate_values"]
    left = a.layers[0].mixer["left"][1]
    assert left["sink"] and left["qk_norm"] == "head" and left["pool"] == 0 and left["out_bias"]
    open_shapes = tensor_shapes(a, nominal=None)
    assert open_shapes["l1.mix.a1"] == (None, 40) and open_shapes["l3.dwa"] == (5,) and "l1.norm2" not in open_shapes
    assert set(open_shapes) == set(W)
    t = resolve_arch("pozalorn-tiny")
    assert t.family == "pozalorn" and t.num_params() > 0


# --------------------------------------------------------------------------------- mechanisms alone
def _step_meta(lens_new, ctx, tables, d):
    """Device tensors of one step: per sequence ``lens_new`` new tokens that end at context ``ctx``."""
    pos, slots, qs = [], [], [0]
    for s, (n, c) in enumerate(zip(lens_new, ctx)):
        for j in range(c - n, c):
            pos.append(j)
            slots.append(int(tables[s][j // 16]) * 16 + j % 16)
        qs.append(qs[-1] + n)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=d)  # noqa: E731
    return i32(pos), i32(slots), i32(qs), i32(ctx)


def _run_window(d, dt, q, k, v, H, G, size, pool, sink, turn, tables, steps, transposed=False, prefill_kernel=0):
    """Feed sequences through window_write / window_pool / window_attn in the given steps
    (``steps``: list of per-sequence new-token counts); returns each sequence's outputs [T, H * V].
    ``transposed``: keep the transposed value copy, which selects the MFMA kernel (GPU, bf16)."""
    from vgate.ops import seq
    S, D, V = len(q), q[0].shape[1] // H, v[0].shape[1] // G
    pages = int(max(max(t) for t in tables)) + 1
    npool = (16 + pool - 1) // pool if pool else 0
    kc = torch.full((pages, G, 16, D), 9.0, dtype=dt, device=d)
    vc = torch.full((pages, G, 16, V), -9.0, dtype=dt, device=d)
    kp = torch.full((pages, G, npool, D), 9.0, dtype=dt, device=d) if pool else None
    vp = torch.full((pages, G, npool, V), -9.0, dtype=dt, device=d) if pool else None
    vt = torch.full((pages, G, V, 16), -9.0, dtype=dt, device=d) if transposed else None
    bt = torch.zeros(S, max(len(t) for t in tables), dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, : len(t)] = torch.tensor(t, dtype=torch.int32)
    bt = bt.to(d)
    vf = seq.rope_inv_freq(V, 30.0, d) if turn else None
    none = torch.zeros(0, device=d)
    done = [0] * S
    outs = [[] for _ in range(S)]
    for new in steps:
        ctx = [done[s] + new[s] for s in range(S)]
        pos, slots, qs, cl = _step_meta(new, ctx, tables, d)
        cat = lambda xs: torch.cat([xs[s][done[s]: ctx[s]] for s in range(S)]).to(d, dt)  # noqa: E731
        T = int(qs[-1])
        qo = torch.zeros(T, H * D, dtype=dt, device=d)
        seq.window_write(cat(q), cat(k), cat(v), None, None, 1e-6, False, pos, slots, none, 0, vf, kc, vc, qo, H, G, vt=vt)
        if pool:
            seq.window_pool(kc, vc, kp, vp, pos, bt, qs, pool)
        o = torch.zeros(T, H * V, dtype=dt, device=d)
        seq.window_attn(qo, kc, vc, kp, vp, bt, cl, qs, o, 0.5, H, size, pool, sink, vf, vt=vt, prefill_kernel=prefill_kernel)
        for s in range(S):
            outs[s].append(o[int(qs[s]): int(qs[s + 1])].float().cpu())
        done = ctx
    return [torch.cat(x) for x in outs]


def _want_window(q, k, v, H, G, size, pool, sink, turn):
    T, D, V = q.shape[0], q.shape[1] // H, v.shape[1] // G
    fv = oracle.frequencies(V, 30.0, None, torch.float32)
    keys, vals, out = [], [], []
    for t in range(T):
        keys.append(k[t].view(G, D))
        vv = v[t].view(G, V)
        vals.append(torch.stack([oracle.turn_pairs(vv[g], t, fv, V) for g in range(G)]) if turn else vv)
        o = oracle.attend(q[t].view(H, D), keys, vals, t, size, pool, 0.5, sink)
        if turn:
            o = torch.stack([oracle.turn_pairs(o[h], -t, fv, V) for h in range(H)])
        out.append(o.reshape(-1))
    return torch.stack(out)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("size,pool", [(20, 0), (20, 6), (16, 16), (33, 24), (5, 1)])
def test_window_attention_edges(device, f32, size, pool):
    """The attention ops alone on crafted keys: for chosen query positions one key is made to dominate
    (it and the query are scaled along a probe direction): the oldest key inside the window, the first
    one outside, the last token of the newest pooled block that is seen and of the first that is not
    yet, a key hundreds back, one at a page border. A wrong edge moves the output by O(1). Run as one
    prompt, as portions cut inside blocks and windows, and token by token over scattered, reused pages;
    with and without a sink and turned values."""
    dt = torch.float32 if f32 else torch.bfloat16
    g = torch.Generator().manual_seed(11)
    H, G, D, V, T = 4, 2, 8, 6, 150
    d = torch.device(device)
    q, k, v = (torch.randn(T, n, generator=g) * 0.4 for n in (H * D, G * D, G * V))
    probe = torch.randn(D, generator=g)
    probe /= probe.norm()
    queries = [149, 140, 131, 120, 97, 64]
    for n, i in enumerate(queries):
        inside, outside = i - size + 1, i - size
        spots = [inside, outside, 3, 16 * 4]
        if pool and i - size >= pool - 1:
            nb = (i - size + 1) // pool          # blocks seen; block nb is the first unseen
            spots += [nb * pool - 1, nb * pool + pool - 1]
        j = spots[n % len(spots)]
        if 0 <= j <= i:
            k[j].view(G, D)[n % G] += 7.0 * probe
        q[i].view(H, D)[(n % G) * (H // G)] += 5.0 * probe
    q, k, v = (x.to(dt).float() for x in (q, k, v))
    sink = torch.tensor([0.3, -1.0, 2.0, 0.0])
    tables = [[7, 2, 9, 4, 11, 0, 5, 13, 1, 8]]
    for use_sink, turn in ((False, False), (True, True)):
        sk = sink if use_sink else None
        want = _want_window(q, k, v, H, G, size, pool, sk, turn)
        skd = sk.to(d) if use_sink else None
        for steps in ([[T]], [[61], [2], [35], [1], [1], [50]], [[T - 40]] + [[1]] * 40):
            # FMA kernel; on the GPU in bf16 also the two MFMA kernels for prompt portions (0: LDS-staged, 1: split)
            for mfma in ([None, 0, 1] if device == "cuda" and not f32 else [None]):
                got = _run_window(d, dt, [q], [k], [v], H, G, size, pool, skd, turn, tables, steps, transposed=mfma is not None,
                                  prefill_kernel=mfma or 0)[0]
                assert rel(got, want) < (3e-5 if f32 else 2e-2), (use_sink, turn, len(steps), mfma)
        # the crafted keys matter: one more or one fewer key in the window moves the answer
        # (with pool 1 every earlier token is seen either way, as itself or as its own block)
        if pool != 1:
            assert rel(_want_window(q, k, v, H, G, size + 1, pool, sk, turn), want) > 0.02
            assert rel(_want_window(q, k, v, H, G, size - 1, pool, sk, turn), want) > 0.02


@pytest.mark.parametrize("device", DEVICES)
def test_window_attention_batch_and_page_reuse(device):
    """Two sequences in one step against each alone; the second takes over pages the first one used
    (stale keys, values and pooled rows in them must not be seen)."""
    g = torch.Generator().manual_seed(12)
    H, G, D, V = 2, 1, 4, 4
    d = torch.device(device)
    mk = lambda T: tuple(torch.randn(T, n, generator=g) for n in (H * D, G * D, G * V))  # noqa: E731
    (qa, ka, va), (qb, kb, vb) = mk(70), mk(37)
    wa, wb = (_want_window(q, k, v, H, G, 10, 4, None, True) for q, k, v in ((qa, ka, va), (qb, kb, vb)))
    got = _run_window(d, torch.float32, [qa, qb], [ka, kb], [va, vb], H, G, 10, 4, None, True,
                      [[3, 1, 4, 0, 2], [6, 5, 7]], [[30, 1], [2, 30], [38, 6]])
    assert rel(got[0], wa) < 3e-5 and rel(got[1], wb) < 3e-5
    # b again on a's pages, from position 0
    got = _run_window(d, torch.float32, [qb], [kb], [vb], H, G, 10, 4, None, True, [[3, 1, 4]], [[20], [17]])
    assert rel(got[0], wb) < 3e-5
    if device == "cuda":   # the MFMA kernel: rows of two sequences, of several tokens and of one
        for kern in (0, 1):
            got = _run_window(d, torch.bfloat16, [qa, qb], [ka, kb], [va, vb], H, G, 10, 4, None, True,
                              [[3, 1, 4, 0, 2], [6, 5, 7]], [[30, 1], [2, 30], [38, 6]], transposed=True, prefill_kernel=kern)
            assert rel(got[0], wa) < 2e-2 and rel(got[1], wb) < 2e-2, kern


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("per_head", [True, False])
@pytest.mark.parametrize("dims", [6, 4, 0])
def test_window_write_norm_and_rotation(device, per_head, dims):
    """Query / key norm (per head or over the whole projection), rotation of fewer dims than the head
    with scaled frequencies, padding rows (slot -1) write nothing."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(13)
    H, G, D, V, T = 3, 1, 6, 5, 7
    d = torch.device(device)
    q, k, v = (torch.randn(T, n, generator=g) for n in (H * D, G * D, G * V))
    qw, kw = torch.randn(D if per_head else H * D, generator=g), torch.randn(D if per_head else G * D, generator=g)
    pos = torch.tensor([0, 1, 2, 40, 41, 1000, 5], dtype=torch.int32)
    slots = torch.tensor([3, 4, 5, 17, 18, 31, -1], dtype=torch.int32)
    scaling = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 20}
    inv = seq.rope_inv_freq(dims, 50.0, d, scaling=scaling)
    fr = oracle.frequencies(dims, 50.0, scaling, torch.float32)
    assert torch.allclose(inv.cpu(), fr, rtol=1e-6) and (dims == 0 or float(fr[-1]) < 50.0 ** (-2.0 * (dims // 2 - 1) / dims))
    kc, vc = torch.full((2, G, 16, D), 7.0, device=d), torch.full((2, G, 16, V), 7.0, device=d)
    qo = torch.zeros(T, H * D, device=d)
    seq.window_write(q.to(d), k.to(d), v.to(d), qw.to(d), kw.to(d), 1e-5, not per_head, pos.to(d), slots.to(d), inv, dims, None,
                     kc, vc, qo, H, G)
    for t in range(T - 1):
        if per_head:
            qn, kn = oracle.rms_unit(q[t].view(H, D), 1e-5) * qw, oracle.rms_unit(k[t].view(G, D), 1e-5) * kw
        else:
            qn, kn = (oracle.rms_unit(q[t], 1e-5) * qw).view(H, D), (oracle.rms_unit(k[t], 1e-5) * kw).view(G, D)
        qn = torch.stack([oracle.turn_pairs(x, int(pos[t]), fr, dims) for x in qn])
        kn = torch.stack([oracle.turn_pairs(x, int(pos[t]), fr, dims) for x in kn])
        assert torch.allclose(qo[t].cpu(), qn.reshape(-1), atol=3e-5), t
        assert torch.allclose(kc[slots[t] // 16, :, slots[t] % 16].cpu(), kn, atol=3e-5), t
        assert torch.allclose(vc[slots[t] // 16, :, slots[t] % 16].cpu(), v[t].view(G, V), atol=1e-6), t
    used = {int(s) for s in slots if s >= 0}
    flat = kc.cpu().permute(0, 2, 1, 3).reshape(32, G, D)
    assert bool((flat[[i for i in range(32) if i not in used]] == 7.0).all())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("D,V", [(5, 9), (32, 8), (48, 64), (80, 20), (130, 4)])
@pytest.mark.parametrize("channel", [True, False])
def test_linear_attention_state_carry_and_slots(device, D, V, channel):
    """The recurrence alone (key size != value size, per-channel gated decay or one constant per head):
    a sequence cut into steps (state carried in its slot) equals one pass and the oracle; a sequence that
    starts at position 0 ignores what a previous owner left in its slot; two sequences in one step."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(14)
    H, n = 2, 29
    d = torch.device(device)
    q, k = (torch.randn(n, H * D, generator=g) * 0.5 for _ in range(2))
    v, gt = (torch.randn(n, H * V, generator=g) for _ in range(2))
    z = torch.randn(n, H * D, generator=g) * 2.0 + 2.0
    decay = torch.tensor([0.9, 0.6])
    tau, qs_ = 3.0, 0.37
    for in_silu, norm_all, gate_silu in ((False, False, True), (True, True, False)):
        nw = torch.randn(H * V if norm_all else V, generator=g)
        act = oracle.silu if in_silu else (lambda x: x)
        a = (torch.sigmoid(z) ** (1.0 / tau)).view(n, H, D) if channel else decay.view(1, H, 1).expand(n, H, D)
        o = torch.stack([oracle.recurrence(act(q).view(n, H, D)[:, h] * qs_, act(k).view(n, H, D)[:, h], act(v).view(n, H, V)[:, h],
                                           a[:, h])[0] for h in range(H)], 1)
        o = (oracle.rms_unit(o.reshape(n, -1), 1e-5) * nw) if norm_all else (oracle.rms_unit(o, 1e-5) * nw).reshape(n, -1)
        want = o * (oracle.silu(gt) if gate_silu else torch.sigmoid(gt))

        def run(cuts, slot, state, cols=0):
            out = torch.zeros(n, H * V, device=d)
            at = 0
            for c in cuts:
                i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=d)  # noqa: E731
                sl = slice(at, at + c)
                seq.linear_attn(q[sl].to(d), k[sl].to(d), v[sl].to(d), gt[sl].to(d), z[sl].to(d) if channel else None,
                                None if channel else decay.to(d), tau, qs_, in_silu, nw.to(d), norm_all, gate_silu, state,
                                i32([slot]), i32([at + c]), i32([0, c]), out[sl], 1e-5, cols_per_lane=cols)
                at += c
            return out.cpu()

        state = torch.full((3, H, D, V), 5.0, device=d)   # garbage a previous owner left
        assert rel(run([n], 1, state), want) < 3e-5
        assert rel(run([3, 1, 1, 9, 2, 13], 2, state), want) < 3e-5
        assert rel(run([3, 1, 1, 9, 2, 13], 0, state, cols=4), want) < 3e-5
        assert bool((state[0, 0, 0, :] != 5.0).all())


@pytest.mark.parametrize("device", DEVICES)
def test_post_norm_add_and_depth_average(device):
    from vgate.ops import seq
    g = torch.Generator().manual_seed(15)
    T, W, L = 5, 21, 3
    d = torch.device(device)
    hist = torch.randn(L + 1, T, W, generator=g).to(d)
    x, y1, y2 = (torch.randn(T, W, generator=g) for _ in range(3))
    w = torch.randn(W, generator=g)
    coef = torch.randn(3, generator=g)
    u = 0.7 * y1 + 1.3 * y2
    r = x + oracle.rms_unit(u, 1e-5) * w
    mix_want = coef[0] * hist[0].cpu() + coef[1] * hist[1].cpu() + coef[2] * r
    mix, act = torch.zeros(T, W, device=d), torch.zeros(T, W, dtype=torch.bfloat16, device=d)
    seq.post_norm_add(x.to(d), y1.to(d), w.to(d), 1e-5, hist[2], s1=0.7, y2=y2.to(d), s2=1.3, act_out=act, hist=hist, planes=3,
                      coef=coef.to(d), mix=mix)
    assert torch.allclose(hist[2].cpu(), r, atol=1e-5) and torch.allclose(mix.cpu(), mix_want, atol=1e-5)
    assert torch.allclose(act.float().cpu(), mix_want, atol=3e-2, rtol=1e-2)
    xin = x.to(d).clone()  # in place, bf16 input, no history
    seq.post_norm_add(xin, y1.to(d, torch.bfloat16), w.to(d), 1e-5, xin)
    assert torch.allclose(xin.cpu(), x + oracle.rms_unit(y1.to(torch.bfloat16).float(), 1e-5) * w, atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
def test_gelu_pair_gemm(device, f32):
    from vgate.ops import seq
    g = torch.Generator().manual_seed(16)
    d = torch.device(device)
    dt = torch.float32 if f32 else torch.bfloat16
    a, w1, w2 = torch.randn(9, 40, generator=g).to(dt), torch.randn(24, 40, generator=g).to(dt) * 0.3, torch.randn(24, 40, generator=g).to(dt) * 0.3
    out = torch.zeros(9, 24, dtype=dt, device=d)
    seq.gemm(a.to(d), w1.to(d), out, w2=w2.to(d), act=seq.ACT_GELU_TANH_MUL)
    want = oracle.gelu_tanh(a.float() @ w1.float().t()) * (a.float() @ w2.float().t())
    assert rel(out, want) < (1e-5 if f32 else 1e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
def test_glu_rows(device, act):
    from vgate.ops import seq
    g = torch.Generator().manual_seed(17)
    d = torch.device(device)
    gu = (torch.randn(7, 48, generator=g) * 2).to(torch.bfloat16)
    out = torch.zeros(5, 24, dtype=torch.bfloat16, device=d)
    seq.glu_rows(gu.to(d), out, seq.ACT_GELU_TANH_MUL if act == "gelu_tanh" else seq.ACT_SILU_MUL)
    a, u = gu[:5, :24].float(), gu[:5, 24:].float()
    want = (oracle.gelu_tanh(a) if act == "gelu_tanh" else oracle.silu(a)) * u
    assert rel(out, want) < 5e-3


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("D,V", [(16, 24), (72, 40)])
def test_linear_attention_long_portions(device, D, V):
    """Portions of hundreds of tokens (on the GPU scanned in parallel chunks with a carry between them): a
    lone sequence from position 0, its continuation from the slot's state, and two unequal sequences in one
    step, all against the token-by-token recurrence. Decays down to ~0.01 per token: a chunk's decay product
    underflows towards zero, which must stay harmless."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(18)
    H = 2
    d = torch.device(device)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=d)  # noqa: E731

    def make(n):
        q, k = (torch.randn(n, H * D, generator=g) * 0.5 for _ in range(2))
        v, gt = (torch.randn(n, H * V, generator=g) for _ in range(2))
        z = torch.randn(n, H * D, generator=g) * 3.0
        return q, k, v, gt, z

    nw = torch.randn(V, generator=g)
    tau = 1.5

    def want(x):
        q, k, v, gt, z = x
        n = q.shape[0]
        a = (torch.sigmoid(z) ** (1.0 / tau)).view(n, H, D)
        o = torch.stack([oracle.recurrence(q.view(n, H, D)[:, h], k.view(n, H, D)[:, h], v.view(n, H, V)[:, h], a[:, h])[0]
                         for h in range(H)], 1)
        return (oracle.rms_unit(o, 1e-5) * nw).reshape(n, -1) * oracle.silu(gt)

    def step(parts, slots, ctx, state, cols=0):
        """parts: per sequence (tensors, first row, rows)."""
        cat = lambda j: torch.cat([x[j][a: a + n] for x, a, n in parts]).to(d)  # noqa: E731
        T = sum(n for _, _, n in parts)
        out = torch.zeros(T, H * V, device=d)
        qs = [0]
        for _, _, n in parts:
            qs.append(qs[-1] + n)
        seq.linear_attn(cat(0), cat(1), cat(2), cat(3), cat(4), None, tau, 1.0, False, nw.to(d), False, True, state,
                        i32(slots), i32(ctx), i32(qs), out, 1e-5, cols_per_lane=cols)
        return out.cpu()

    A, B = make(700), make(90)
    wa, wb = want(A), want(B)
    for cols in (0, 1, 4):   # columns a lane of the GPU scan keeps (0: by the launch's size)
        state = torch.full((3, H, D, V), 3.0, device=d)
        o1 = step([(A, 0, 450)], [2], [450], state, cols)                       # lone sequence, chunked on the GPU
        o2 = step([(A, 450, 200), (B, 0, 90)], [2, 0], [650, 90], state, cols)  # continuation beside a new sequence
        o3 = step([(A, 650, 50)], [2], [700], state, cols)                      # short step: one pass from the slot
        assert rel(torch.cat([o1, o2[:200], o3]), wa) < 5e-5, cols
        assert rel(o2[200:], wb) < 5e-5, cols
