"""Zadirax (layered hybrid: latent attention, generalized delta rule, gated residual, MoE) in the engine,
against the plain implementation of tests/zadirax_oracle.py.

Small configurations with random weights are written to a temporary folder (config.json +
model.safetensors) and run through ``LLMEngine.replay_step`` / ``add_request`` on the CPU device
(unfused torch forms of the ops) and, marked ``gpu``, on the HIP kernels, in fp32 and bf16.
"""
from __future__ import annotations

import json
import math

import pytest
import torch

import zadirax_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


# ------------------------------------------------------------------------------------ configurations
def _delta(H, D, mlp, **kw):
    return {"type": "general_delta", "mixer": {"heads": H, "dim": D}, "mlp": mlp, **kw}


def _latent(H, D, R, V, KR, QR, mlp, base=10000.0, **kw):
    return {"type": "latent_attention",
            "mixer": {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": KR, "q_rank": QR,
                      "rot": {"base": base, "dims": R}, "scale": 1.0 / math.sqrt(D + R)}, "mlp": mlp, **kw}


def _moe(E, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": E, "top": top}}


def config_a():
    moe = _moe(4, 2, 10, 1.5)
    lat = _latent(3, 8, 4, 6, 20, 12, moe)
    return {"architecture": "Zadirax", "width": 40, "vocab": 50, "norm": {"eps": 1e-5},
            "layers": [_delta(2, 12, {"kind": "dense", "ff": 24}), lat, _delta(2, 12, None), dict(lat, weights_of=1)]}


def config_b():
    """Sizes that make things equal or 1: one head, top 1, value size = key size, latent first."""
    lat = _latent(1, 4, 2, 4, 8, 8, {"kind": "dense", "ff": 8}, base=100.0)
    return {"architecture": "Zadirax", "width": 24, "vocab": 30, "norm": {"eps": 1e-6},
            "layers": [lat, _delta(1, 5, _moe(3, 1, 6, 0.7)), dict(lat, weights_of=0), _delta(3, 7, None)]}


def config_c():
    """Sizes in the range the fragment-packed MFMA GEMMs take (width 512, multiples of 64)."""
    lat = _latent(4, 64, 64, 64, 192, 128, _moe(6, 2, 128, 3.0))
    return {"architecture": "Zadirax", "width": 512, "vocab": 640, "norm": {"eps": 1e-6},
            "layers": [_delta(4, 64, {"kind": "dense", "ff": 512}), lat, _delta(2, 128, {"kind": "dense", "ff": 512})]}


def config_d():
    """Awkward sizes: a latent that is not a whole number of 16-column tiles, five heads, head sizes of the
    recurrence that fill their key groups unevenly, every expert chosen, a vocabulary that is not a multiple of 4."""
    lat = _latent(5, 24, 8, 40, 136, 48, _moe(3, 3, 24, 1.0), base=500.0)
    return {"architecture": "Zadirax", "width": 72, "vocab": 101, "norm": {"eps": 1e-6},
            "layers": [lat, _delta(3, 40, None), _delta(2, 100, {"kind": "dense", "ff": 50}), dict(lat, weights_of=0)]}


def make_tensors(cfg: dict, seed: int, decay_rank: int = 3) -> dict:
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.5):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    t = {"embed": (torch.randn(V, W, generator=g)).to(torch.bfloat16), "head": mat(V, W), "final.norm": vec((), 1.2, 0.0)}
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = vec((), 0.9, 0.0)
        t[p + "rg1"], t[p + "rg1.b"] = mat(W, W), vec(W)
        if L["type"] == "latent_attention":
            H, D, R, Vd, KR, QR = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            t.update({p + "mix.dq": mat(QR, W), p + "mix.dq.norm": vec(QR, 1.0, 0.2), p + "mix.uq": mat(H * (D + R), QR, 2.0),
                      p + "mix.dkv": mat(KR + R, W, 2.0), p + "mix.dkv.norm": vec(KR, 1.0, 0.2), p + "mix.uk": mat(H * D, KR, 2.0),
                      p + "mix.uv": mat(H * Vd, KR), p + "mix.g": mat(H * Vd, W), p + "mix.o": mat(W, H * Vd)})
        else:
            n = m["heads"] * m["dim"]
            t.update({p + "mix." + k: mat(n, W) for k in ("r", "k", "v", "g", "a")})
            t.update({p + "mix.a.b": vec(n), p + "mix.w1": mat(decay_rank, W), p + "mix.w2": mat(n, decay_rank, 2.0),
                      p + "mix.w0": vec(n, 0.0, 1.0), p + "mix.norm": vec(n, 1.0, 0.2), p + "mix.o": mat(W, n)})
        f = L.get("mlp")
        if f:
            t[p + "rg2"], t[p + "rg2.b"] = mat(W, W), vec(W)
            if f["kind"] == "dense":
                t.update({p + "mlp.gate": mat(f["ff"], W), p + "mlp.up": mat(f["ff"], W), p + "mlp.down": mat(W, f["ff"])})
            else:
                E, ff = f["router"]["experts"], f["expert"]["ff"]
                t[p + "mlp.router"], t[p + "mlp.correction"] = mat(E, W, 3.0), vec(E, 0.0, 0.3)
                for e in range(E):
                    t.update({p + f"mlp.e{e}.gate": mat(ff, W, 2.0), p + f"mlp.e{e}.up": mat(ff, W, 2.0),
                              p + f"mlp.e{e}.down": mat(W, ff)})
    return t


_MODELS: dict = {}


def model_dir(tmp_path_factory, name: str):
    """(folder, config dict, fp32 tensors) of a named test model, written once per session."""
    if name not in _MODELS:
        from safetensors.torch import save_file
        cfg = {"a": config_a, "b": config_b, "c": config_c, "d": config_d}[name]()
        t = make_tensors(cfg, seed=11 if name == "a" else 23, decay_rank=3 if name == "a" else 2)
        d = tmp_path_factory.mktemp("zadirax_" + name)
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
@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_whole_prompt_matches_oracle(tmp_path_factory, device, dtype, name):
    path, cfg, W = model_dir(tmp_path_factory, name)
    toks = tokens_of(cfg, 37, seed=1)
    eng = engine(path, device, dtype)
    lg = replay_all(eng, "w", toks, [len(toks)])
    assert rel(lg, oracle_logits(name, cfg, W, toks)) < tol(dtype)
    one = replay_all(eng, "one", toks[:1], [1])  # a sequence of one token (first position only)
    assert rel(one, oracle_logits(name, cfg, W, toks)[:1]) < tol(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_oracle(tmp_path_factory, device):
    path, cfg, W = model_dir(tmp_path_factory, "a")
    toks = tokens_of(cfg, 19, seed=2)
    eng = engine(path, device, "float32")
    eng.model.capture_layers = []
    replay_all(eng, "l", toks, [len(toks)])
    want: list = []
    oracle.forward(cfg, W, toks, want)
    assert len(eng.model.capture_layers) == len(want) == len(cfg["layers"])
    for i, (got, w) in enumerate(zip(eng.model.capture_layers, want)):
        assert rel(got[: len(toks)], w) < 1e-4, f"residual stream after layer {i}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[1], [20], [2, 2, 2, 3, 5, 7, 16, 17], [15, 1, 16, 2, 14], [33, 2]])
def test_portions_and_decoding_match_whole(tmp_path_factory, device, dtype, cuts):
    """Prefill against token-by-token decoding and portions of several sizes down to two tokens (cuts
    inside pages and at their borders); the tail decodes one token at a time (long decoding)."""
    path, cfg, W = model_dir(tmp_path_factory, "a")
    toks = tokens_of(cfg, 70, seed=3)
    eng = engine(path, device, dtype)
    whole = replay_all(eng, "whole", toks, [len(toks)])
    cut = replay_all(eng, "cut", toks, cuts)
    assert rel(cut, whole) < (2e-5 if dtype == "float32" else 3e-2)
    assert rel(cut, oracle_logits("a", cfg, W, toks)) < tol(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_and_reuse(tmp_path_factory, device, dtype):
    """Unequal requests in one batch (portions beside single tokens) against each alone, with a pool
    so small that pages and state slots are freed and taken again by later requests."""
    path, cfg, W = model_dir(tmp_path_factory, "a")
    reqs = {f"q{i}": tokens_of(cfg, n, seed=10 + i) for i, n in enumerate([41, 5, 23, 1, 30, 17, 9])}
    eng = engine(path, device, dtype, pages=8, seqs=3)  # 128 tokens, 3 slots: 7 requests must reuse both
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
        assert rel(torch.cat(got[k]), oracle_logits("a", cfg, W, toks)) < tol(dtype), k


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_awkward_sizes_portions_and_batches(tmp_path_factory, device, dtype):
    path, cfg, W = model_dir(tmp_path_factory, "d")
    ta, tb = tokens_of(cfg, 45, seed=7), tokens_of(cfg, 21, seed=8)
    eng = engine(path, device, dtype)
    got_a, got_b = [], []
    plan = [([0, 17], [0, 1]), ([17, 19], [1, 2]), ([19, 40], [2, 21]), ([40, 41], None), ([41, 45], None)]
    for (a0, a1), br in plan:
        entries = [("A", ta[a0:a1], list(range(a1 - a0)))]
        if br:
            entries.append(("B", tb[br[0]:br[1]], list(range(br[1] - br[0]))))
        lg = eng.replay_step(entries, (["A"] if a1 == 45 else []) + (["B"] if br and br[1] == 21 else [])).float().cpu()
        got_a.append(lg[: a1 - a0])
        if br:
            got_b.append(lg[a1 - a0:])
    assert rel(torch.cat(got_a), oracle_logits("d", cfg, W, ta)) < tol(dtype)
    assert rel(torch.cat(got_b), oracle_logits("d", cfg, W, tb)) < tol(dtype)


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
    path, cfg, W = model_dir(tmp_path_factory, "a")
    eng = engine(path, "cuda", "bfloat16", pages=32, seqs=4, enforce_eager=False)
    outs = []
    for rnd in range(2):
        done = {}
        for i in range(3):
            eng.add_request(f"r{rnd}_{i}", prompt_ids=tokens_of(cfg, 9 + 7 * i, seed=40 + i),
                            params=SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True),
                            callback=lambda kind, seq, payload: done.__setitem__(seq.request_id[3:], seq.output_ids))
        hits = eng.runner.graph_hits
        eng.run_until_idle()
        outs.append(done)
    assert eng.runner.graph_hits > hits
    assert outs[0] == outs[1]


@pytest.mark.gpu
def test_packed_gemm_path_matches_row_major_and_oracle(tmp_path_factory, monkeypatch):
    """bf16 at sizes whose projections run on the fragment-packed MFMA GEMMs: same logits as with every
    matrix on the row-major GEMM, and the oracle's; prompt portions, decoded tokens and a second request."""
    from vgate.models import mixers
    path, cfg, W = model_dir(tmp_path_factory, "c")
    toks = tokens_of(cfg, 45, seed=5)
    got = {}
    for packed in (True, False):
        monkeypatch.setattr(mixers, "USE_PACKED", packed)
        eng = engine(path, "cuda", "bfloat16")
        assert eng.model.layers[0].proj.packed == packed and eng.model.head.packed == packed
        got[packed] = replay_all(eng, "p", toks, [30, 2, 9])
        del eng
    assert rel(got[True], got[False]) < 2e-2
    # (bf16 rounding alone moves this model's logits by ~0.09 of their size; fp32 below is the sharp check)
    assert rel(got[True], oracle_logits("c", cfg, W, toks)) < 0.2
    eng = engine(path, "cuda", "float32")
    assert rel(replay_all(eng, "f", toks, [30, 2, 9]), oracle_logits("c", cfg, W, toks)) < tol("float32")


def test_registry_and_config():
    from vgate.models.config import HybridArch, resolve_arch
    from vgate.models.hybrid import tensor_shapes
    a = resolve_arch("zadirax-tiny")
    assert isinstance(a, HybridArch) and a.family == "zadirax" and a.owner(3) == 1
    names = tensor_shapes(a)
    assert "l1.mix.dkv" in names and "l3.mix.dkv" not in names and names["l0.norm1"] == ()
    assert a.num_params() == sum(math.prod(s) for s in names.values())
    with pytest.raises(ValueError):
        from vgate.models import build_model
        build_model(resolve_arch("tiny"), "cpu", dtype="float32")


def test_state_slots_follow_pages():
    from vgate.runtime.kv_cache import KVCacheManager
    from vgate.runtime.sampling_params import SamplingParams
    from vgate.runtime.sequence import Sequence
    kvm = KVCacheManager(8, 16, False, prefer_native=False, state_slots=2)
    s = [Sequence(request_id=str(i), prompt_ids=[1] * 20, params=SamplingParams()) for i in range(3)]
    assert kvm.ensure(s[0], 20) and kvm.ensure(s[1], 20)
    assert {s[0].state_slot, s[1].state_slot} == {0, 1}
    assert not kvm.ensure(s[2], 20) and s[2].state_slot == -1 and not s[2].blocks  # no slot: nothing taken
    kvm.free(s[0])
    assert s[0].state_slot == -1 and kvm.ensure(s[2], 20) and s[2].state_slot in (0, 1)


# --------------------------------------------------------------------------------- mechanisms alone
def _dev(device):
    return torch.device(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
def test_latent_attention_far_keys_and_edges(device, f32):
    """The attention op alone on a crafted cache: several hundred keys over scattered pages, ONE far key
    (and one at a page border) made to dominate by scaling it and the query, a dominating key placed just
    AFTER a query's position (must not be seen) and one exactly AT it (must be)."""
    from vgate.ops import seq
    dt = torch.float32 if f32 else torch.bfloat16
    g = torch.Generator().manual_seed(5)
    H, rank, rot, page = 3, 24, 6, 16
    E = rank + rot
    ctx, nq = 331, 6                       # the step brings the last 6 tokens of a 331-token sequence
    rows = torch.randn(ctx, E, generator=g) * 0.3
    qa = torch.randn(nq, H, E, generator=g) * 0.3
    probe = torch.randn(E, generator=g)
    probe = probe / probe.norm()
    far, border = 7, 16 * 9                # a key hundreds back, and the first row of a page
    rows[far] += 6.0 * probe
    rows[border] += 5.0 * probe
    rows[ctx - nq + 2] += 9.0 * probe      # query 2's own position: visible to it and later ones only
    qa[:, 0] += 4.0 * probe                # head 0 looks for the probe direction
    rows, qa = rows.to(dt), qa.to(dt)
    nblk = (ctx + page - 1) // page
    perm = torch.randperm(40, generator=g)[:nblk]
    cache = torch.zeros(40, page, E, dtype=dt)
    for j in range(ctx):
        cache[perm[j // page], j % page] = rows[j]
    cache[perm[(ctx - 1) // page], (ctx - 1) % page + 1:] = 50.0   # stale rows after the last token
    bt = torch.zeros(1, 24, dtype=torch.int32)
    bt[0, :nblk] = perm.int()
    d = _dev(device)
    want = oracle_attend(qa.float(), rows.float(), rank, 0.7, ctx - nq)
    # bf16 on the GPU: also with the transposed copy of the latent part, which selects the MFMA kernel
    copies = [None] if f32 or device == "cpu" else [None, cache[:, :, :rank].transpose(1, 2).contiguous().to(d)]
    for cache_t in copies:
        ol = torch.zeros(nq, H, rank, dtype=dt, device=d)
        seq.latent_attn(qa.to(d), cache.to(d), bt.to(d), torch.tensor([ctx], dtype=torch.int32, device=d),
                        torch.tensor([0, nq], dtype=torch.int32, device=d), ol, 0.7, H, rank, rot, cache_t=cache_t)
        assert rel(ol, want) < (2e-5 if f32 else 1e-2), "mfma" if cache_t is not None else "fma"
    # the crafted keys matter: without the far key, or seeing the key one place too far, the answer moves
    no_far = rows.float().clone()
    no_far[far] -= 6.0 * probe
    assert rel(oracle_attend(qa.float(), no_far, rank, 0.7, ctx - nq), want) > 0.05
    assert rel(oracle_attend(qa.float(), rows.float(), rank, 0.7, ctx - nq + 1), want) > 0.05


def oracle_attend(qa, rows, rank, scale, first_pos):
    out = torch.zeros(qa.shape[0], qa.shape[1], rank)
    for i in range(qa.shape[0]):
        vis = rows[: first_pos + i + 1]
        for h in range(qa.shape[1]):
            p = torch.softmax((vis @ qa[i, h]) * scale, 0)
            out[i, h] = p @ vis[:, :rank]
    return out


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [6, 4, 0])
def test_latent_write_rotation_and_norm(device, dims):
    """Latent norm + rotation of the shared key part + paged store; rotated leading dims may be fewer
    than the part's size (the rest passes unchanged); padding tokens (slot -1) write nothing."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(6)
    rank, rot, T = 10, 6, 9
    kv = torch.randn(T, rank + rot + 3, generator=g)
    w = torch.randn(rank, generator=g)
    pos = torch.tensor([0, 1, 2, 40, 41, 1000, 5, 0, 0], dtype=torch.int32)
    slots = torch.tensor([3, 4, 5, 17, 18, 31, 9, -1, -1], dtype=torch.int32)
    d = _dev(device)
    cache = torch.full((2, 16, rank + rot), 7.0, device=d)
    inv = seq.rope_inv_freq(dims, 50.0, d)
    seq.latent_write(kv.to(d)[:, 3:], w.to(d), 1e-5, pos.to(d), slots.to(d), inv, dims, cache, rank)
    flat = cache.view(-1, rank + rot).cpu()
    for t in range(T):
        if slots[t] < 0:
            continue
        c = oracle.unit_rms(kv[t, 3: 3 + rank], 1e-5) * w
        kr = kv[t, 3 + rank:].clone()
        for i in range(dims // 2):
            ang = torch.tensor(float(pos[t])) * torch.tensor(50.0) ** (-2.0 * i / dims)
            a, b = kr[2 * i].clone(), kr[2 * i + 1].clone()
            kr[2 * i], kr[2 * i + 1] = a * torch.cos(ang) - b * torch.sin(ang), b * torch.cos(ang) + a * torch.sin(ang)
        assert torch.allclose(flat[slots[t]], torch.cat([c, kr]), atol=2e-5), t
    untouched = [i for i in range(32) if i not in slots.tolist()]
    assert bool((flat[untouched] == 7.0).all())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("D", [5, 48, 64, 80])
def test_delta_rule_state_carry_and_slots(device, D):
    """The recurrence alone: a sequence cut into steps (state carried in its slot) equals one pass; a
    sequence that starts at position 0 ignores what a previous owner left in its slot."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(7)
    H, n = 2, 13
    hd = H * D
    P = torch.randn(n, 5 * hd, generator=g)
    wl = torch.randn(n, hd, generator=g)
    w0, ab, nw = (torch.randn(hd, generator=g) for _ in range(3))
    d = _dev(device)

    def run(cuts, slot, state):
        out = torch.zeros(n, hd, device=d)
        at = 0
        for c in cuts:
            sl = slice(at, at + c)
            Pd = P[sl].to(d)
            seq.delta_rule(*(Pd[:, i * hd:(i + 1) * hd] for i in range(5)), wl[sl].to(d).contiguous(), w0.to(d), ab.to(d),
                           nw.to(d), state, torch.tensor([-1, slot], dtype=torch.int32, device=d),
                           torch.tensor([0, at + c], dtype=torch.int32, device=d),
                           torch.tensor([0, 0, c], dtype=torch.int32, device=d), out[sl], 0.55, 1e-6, 1e-5, num_seqs=2)
            at += c
        return out.cpu()

    state = torch.randn(3, H, D, D, generator=g).to(d) * 5.0   # garbage of earlier owners
    one = run([n], 1, state)
    cut = run([1, 2, 7, 1, 2], 2, state)
    assert rel(cut, one) < 1e-5
    # plain recurrence
    r, k, v, gg, a = (P[:, i * hd:(i + 1) * hd].reshape(n, H, D) for i in range(5))
    dec = torch.exp(-0.55 * oracle.sigmoid(wl + w0)).reshape(n, H, D)
    rate = oracle.sigmoid(a + ab.reshape(H, D))
    want = torch.zeros(n, H, D)
    for h in range(H):
        S = torch.zeros(D, D)
        for t in range(n):
            u = k[t, h] / torch.sqrt((k[t, h] ** 2).sum() + 1e-6)
            S = dec[t, h][:, None] * S - torch.outer(rate[t, h] * u, u @ S) + torch.outer(k[t, h], v[t, h])
            want[t, h] = S.T @ r[t, h]
    want = (oracle.unit_rms(want, 1e-5) * nw.reshape(H, D) * oracle.sigmoid(gg)).reshape(n, hd)
    assert rel(one, want) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
def test_moe_choice_uses_correction_weights_do_not(device):
    from vgate.ops import seq
    d = _dev(device)
    z = torch.tensor([[2.0, 1.0, -1.0, 0.5], [0.0, 0.1, 0.2, 0.3]])
    corr = torch.tensor([-5.0, 0.0, 3.0, 0.0])
    idx = torch.empty(2, 2, dtype=torch.int32, device=d)
    wts = torch.empty(2, 2, device=d)
    seq.moe_route(z.to(d), corr.to(d), 2, 1e-20, idx, wts)
    s = oracle.sigmoid(z)
    assert sorted(idx[0].tolist()) == [1, 2] and sorted(idx[1].tolist()) == [2, 3]   # expert 0 loses by its correction
    for t in range(2):
        chosen = idx[t].tolist()
        assert torch.allclose(wts[t].cpu(), s[t, chosen] / s[t, chosen].sum(), atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
def test_row_major_gemm_forms(device, f32):
    """Odd sizes, per-head batches over strided views, gated pairs, expert groups of unequal (and empty) size."""
    from vgate.ops import seq
    d = _dev(device)
    dt = torch.float32 if f32 else torch.bfloat16
    g = torch.Generator().manual_seed(8)
    t = 2e-5 if f32 else 1.5e-2
    a = torch.randn(70, 37, generator=g).to(dt)
    w = torch.randn(29, 37, generator=g).to(dt)
    out = torch.empty(70, 29, dtype=dt, device=d)
    seq.gemm(a.to(d), w.to(d), out, act=seq.ACT_TANH)
    assert rel(out, torch.tanh(a.float() @ w.float().T)) < t
    # wide aligned outputs (the 128-column block tile on the GPU), single matrix + bias and a SiLU pair
    a2 = torch.randn(300, 72, generator=g).to(dt)
    w2a, w2b = (torch.randn(520, 72, generator=g) / 8).to(dt), (torch.randn(520, 72, generator=g) / 8).to(dt)
    bias = torch.randn(520, generator=g)
    o2 = torch.empty(300, 520, dtype=dt, device=d)
    seq.gemm(a2.to(d), w2a.to(d), o2, bias=bias.to(d))
    assert rel(o2, a2.float() @ w2a.float().T + bias) < t
    seq.gemm(a2.to(d), w2a.to(d), o2, w2=w2b.to(d), act=seq.ACT_SILU_MUL)
    ga = a2.float() @ w2a.float().T
    assert rel(o2, ga * oracle.sigmoid(ga) * (a2.float() @ w2b.float().T)) < t
    # per head, reading and writing slices of wider rows
    q = torch.randn(9, 3, 11, generator=g).to(dt)
    wh = torch.randn(3, 6, 7, generator=g).to(dt)
    o = torch.zeros(9, 3, 10, dtype=dt, device=d)
    seq.gemm(q.to(d)[:, :, :7].permute(1, 0, 2), wh.to(d), o[:, :, :6].permute(1, 0, 2))
    assert rel(o[:, :, :6], torch.einsum("thk,hnk->thn", q.float()[:, :, :7], wh.float())) < t
    assert bool((o[:, :, 6:] == 0).all())
    # experts: rows gathered and grouped on the device, clamped gated activation
    E, T, K, N = 4, 21, 18, 13
    tok_e = torch.tensor([0, 2, 2, 2, 0, 2, 3] * 3)      # expert 1 gets nothing
    idx = tok_e[:, None].int()
    rows, pos, off = (torch.empty(n, dtype=torch.int32, device=d) for n in (T, T, E + 1))
    seq.moe_sort(idx.to(d), E, rows, pos, off)
    assert off.tolist() == [0, 6, 6, 18, 21]
    h = torch.randn(T, K, generator=g).to(dt)
    wg, wu = torch.randn(E, N, K, generator=g).to(dt), torch.randn(E, N, K, generator=g).to(dt)
    y = torch.empty(T, N, dtype=dt, device=d)
    seq.gemm(h.to(d), wg.to(d), y, w2=wu.to(d), a_rows=rows, group_off=off, act=seq.ACT_CLAMPED_GLU, limit=0.8)
    back = torch.empty(T, N, dtype=dt, device=d)
    seq.moe_combine(y, pos, torch.ones(T, 1, device=d), back)
    gg = torch.einsum("tk,tnk->tn", h.float(), wg.float()[tok_e]).clamp(max=0.8)
    uu = torch.einsum("tk,tnk->tn", h.float(), wu.float()[tok_e]).clamp(-0.8, 0.8)
    assert rel(back, gg * oracle.sigmoid(1.702 * gg) * (uu + 1)) < t
