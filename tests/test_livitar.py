"""Livitar (tanh-norm layers over several learned-weight copies of the stream; retention; full causal
attention whose positions enter as a distance term of the score; softmax-routed experts with a shared
one) in the engine, against the plain implementation of tests/livitar_oracle.py.

Small configurations with random weights are written to a temporary folder (config.json +
model.safetensors) and run through ``LLMEngine.replay_step`` / ``add_request`` on the CPU device
(unfused torch forms of the ops) and, marked ``gpu``, on the HIP kernels, in fp32 and bf16.
"""
from __future__ import annotations

import json
import math

import pytest
import torch

import livitar_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


# ------------------------------------------------------------------------------------ configurations
def _moe(experts, top, ff, shared, scale=1.7):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def _ret(H, D, V, dims, base, decay, mlp):
    return {"type": "retention", "mlp": mlp,
            "mixer": {"heads": H, "dim": D, "vdim": V, "rot": {"base": base, "dims": dims}, "decay": decay}}


def _att(H, G, D, V, mlp, scale=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale or 1.0 / math.sqrt(D)}}


def _att2(H, G, D, V, far, coef, every, mlp, scale=None):
    return {"type": "attention_2", "mlp": mlp,
            "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale or 2.0 / math.sqrt(D), "bias_max": far,
                      "q_temp": {"coef": coef, "every": every}}}


def config_a():
    """Unequal everything: three copies of the stream, key size != value size, fewer rotated dims than the
    head, a distance table with an odd number of rows, a layer without feed-forward, attention first, a
    vocabulary that is not a multiple of 4."""
    return {"architecture": "Livitar", "width": 40, "vocab": 50, "streams": 3, "norm": {"eps": 1e-5}, "layers": [
        _att2(6, 3, 8, 6, 21, 0.4, 5, _moe(5, 2, 12, 20)),
        _ret(3, 10, 6, 6, 100.0, [0.5, 0.9, 0.995], None),
        _att(4, 2, 12, 10, _moe(5, 2, 12, 20)),
        _ret(2, 6, 12, 6, 10000.0, [0.97, 0.8], _moe(3, 3, 16, None))]}


def config_b():
    """Values that are 1 or equal: one copy of the stream, one head everywhere, one expert of which one is
    chosen, a table of two rows, a query temperature that grows at every position, no decay at all."""
    return {"architecture": "Livitar", "width": 24, "vocab": 32, "streams": 1, "norm": {"eps": 1e-6}, "layers": [
        _ret(1, 4, 4, 4, 10.0, [1.0], _moe(1, 1, 8, None, scale=1.0)),
        _att2(1, 1, 4, 4, 3, 1.0, 1, _moe(2, 1, 8, 8)),
        _att(1, 1, 6, 5, None)]}


def config_c():
    """Page-scale geometry: distance tables that end inside the second page and after the sixth, temperatures
    that step at page borders and inside pages, four copies of the stream, every expert chosen."""
    return {"architecture": "Livitar", "width": 64, "vocab": 96, "streams": 4, "norm": {"eps": 1e-6}, "layers": [
        _ret(2, 16, 24, 16, 10000.0, [0.9, 0.999], _moe(4, 4, 24, 32)),
        _att2(4, 2, 16, 32, 30, 0.25, 16, _moe(6, 2, 24, 32)),
        _att(2, 2, 32, 16, _moe(6, 2, 24, 32)),
        _att2(4, 1, 24, 8, 100, 0.5, 7, _moe(6, 3, 24, None))]}


def config_d():
    """Sizes in the range the fragment-packed MFMA GEMMs take (width 512, projections in multiples of 64)."""
    return {"architecture": "Livitar", "width": 512, "vocab": 704, "streams": 2, "norm": {"eps": 1e-6}, "layers": [
        _ret(4, 64, 64, 64, 10000.0, [0.9, 0.97, 0.99, 0.999], _moe(4, 2, 128, 512)),
        _att(8, 2, 64, 64, _moe(4, 2, 128, 512)),
        _att2(4, 2, 64, 128, 60, 0.2, 32, _moe(4, 2, 128, 512))]}


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d}
TABLE_ROWS = {"a": 7, "b": 2, "c": 16, "d": 12}


def make_tensors(cfg: dict, seed: int, rows: int) -> dict:
    g = torch.Generator().manual_seed(seed)
    W, V, S = cfg["width"], cfg["vocab"], cfg["streams"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.5):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    def pos(n, lo, hi):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(torch.bfloat16)

    def norm(p):
        return {p: vec(W, 1.0, 0.3), p + ".b": vec(W, 0.0, 0.2), p + ".alpha": pos(1, 0.4, 1.2).reshape(())}

    def hyper(p):
        return {p + "in": vec(S, 1.0 / S, 0.3), p + "out": vec(S, 1.0, 0.4),
                p + "mix": (torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)).to(torch.bfloat16)}

    def gated(p, f):
        return {p + "gate": mat(f, W, 2.0), p + "up": mat(f, W), p + "down": mat(W, f)}

    t = {"embed": torch.randn(V, W, generator=g).to(torch.bfloat16), "head": mat(V, W)}
    t.update(norm("final.norm"))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t.update(norm(p + "norm1"))
        t.update(hyper(p + "hc1."))
        H, D, Vd = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        x = p + "mix."
        t.update({x + "q": mat(H * D, W, 2.0), x + "k": mat(G * D, W, 2.0), x + "v": mat(G * Vd, W), x + "g": mat(H * Vd, W, 2.0),
                  x + "o": mat(W, H * Vd)})
        if L["type"] == "attention":
            t.update({x + "temp": pos(H, 0.5, 2.0), x + "r1": pos(H, 0.1, 1.5), x + "r2": pos(H, 0.05, 2.0)})
        elif L["type"] == "attention_2":
            t[x + "rel"] = (1.5 * torch.randn(rows, H, generator=g)).to(torch.bfloat16)
        if L.get("mlp"):
            f = L["mlp"]
            t.update(norm(p + "norm2"))
            t.update(hyper(p + "hc2."))
            t[p + "mlp.router"] = mat(f["router"]["experts"], W, 3.0)
            for e in range(f["router"]["experts"]):
                t.update(gated(f"{p}mlp.e{e}.", f["expert"]["ff"]))
            if f.get("shared"):
                t.update(gated(p + "mlp.shared.", f["shared"]["ff"]))
    return t


_MODELS: dict = {}


def model_dir(tmp_path_factory, name: str):
    """(folder, config dict, fp32 tensors) of a named test model, written once per session."""
    if name not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]()
        t = make_tensors(cfg, seed={"a": 3, "b": 5, "c": 7, "d": 9}[name], rows=TABLE_ROWS[name])
        d = tmp_path_factory.mktemp("livitar_" + name)
        save_file({k: v.contiguous() for k, v in t.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[name] = (str(d), cfg, {k: v.float() for k, v in t.items()})
    return _MODELS[name]


_ORACLE: dict = {}


def oracle_logits(name, cfg, W, tokens):
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = oracle.forward(cfg, W, list(tokens))[0].float()
    return _ORACLE[key]


def engine(path, device, dtype, pages=16, seqs=4, **kw):
    from vgate.runtime.engine import EngineConfig, LLMEngine
    cfg = dict(model=path, dtype=dtype, device=device, max_model_len=pages * 16, max_num_seqs=seqs,
               max_num_batched_tokens=pages * 16, num_kv_blocks=pages, enable_prefix_caching=False, enforce_eager=True,
               warmup=False, prefill_autotune=False, async_scheduling=False)
    cfg.update(kw)
    return LLMEngine(EngineConfig(**cfg))


def rel(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt())


def tol(dtype: str) -> float:
    return 3e-4 if dtype == "float32" else 6e-2


def close(got: torch.Tensor, want: torch.Tensor, dtype: str) -> bool:
    """fp32: the whole result within tol. bf16: rounding can turn a router's close call at a single token,
    which moves that token's logits by O(1) in models this small; so per token, the median within tol and four
    in five within 0.15 (a fault of a mechanism moves most tokens by O(1))."""
    if dtype == "float32":
        return rel(got, want) < tol(dtype)
    g, w = got.double().cpu(), want.double().cpu()
    e = (g - w).pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
    return float(e.median()) < tol(dtype) and float((e < 0.15).double().mean()) >= 0.8


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
    assert close(lg, oracle_logits(name, cfg, W, toks), dtype)
    one = replay_all(eng, "one", toks[:1], [1])  # a sequence of one token (first position only)
    assert close(one, oracle_logits(name, cfg, W, toks)[:1], dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_layers_match_oracle(tmp_path_factory, device, name):
    path, cfg, W = model_dir(tmp_path_factory, name)
    toks = tokens_of(cfg, 23, seed=2)
    eng = engine(path, device, "float32")
    eng.model.capture_layers = []
    replay_all(eng, "l", toks, [len(toks)])
    want: list = []
    oracle.forward(cfg, W, toks, per_layer=want)
    assert len(eng.model.capture_layers) == len(want) == len(cfg["layers"])
    for i, (got, w) in enumerate(zip(eng.model.capture_layers, want)):
        assert rel(got[: len(toks)], w) < 1e-4, f"sum of the stream's copies after layer {i}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[1], [30], [2, 2, 2, 3, 5, 7, 16, 17], [15, 1, 16, 2, 14], [47, 2]])
def test_portions_and_decoding_match_whole(tmp_path_factory, device, dtype, cuts):
    """Prefill against token-by-token decoding and portions of several sizes down to two tokens (cuts inside
    pages and at their borders, across the distance tables' last rows and the temperatures' steps); the
    tail decodes one token at a time."""
    path, cfg, W = model_dir(tmp_path_factory, "c")
    toks = tokens_of(cfg, 120, seed=3)
    eng = engine(path, device, dtype)
    whole = replay_all(eng, "whole", toks, [len(toks)])
    cut = replay_all(eng, "cut", toks, cuts)
    assert rel(cut, whole) < 2e-5 if dtype == "float32" else close(cut, whole, dtype)
    assert close(cut, oracle_logits("c", cfg, W, toks), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(tmp_path_factory, device):
    """A short prompt and then hundreds of single tokens: the recurrent state and the caches carry everything."""
    path, cfg, W = model_dir(tmp_path_factory, "a")
    toks = tokens_of(cfg, 300, seed=4)
    eng = engine(path, device, "float32", pages=20)
    got = replay_all(eng, "d", toks, [3])
    want = oracle_logits("a", cfg, W, toks)
    assert rel(got, want) < tol("float32") and rel(got[-5:], want[-5:]) < tol("float32")


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
        assert close(torch.cat(got[k]), oracle_logits(name, cfg, W, toks), dtype), k


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
    """bf16 at sizes whose projections run on the fragment-packed MFMA GEMMs: same logits as with every
    matrix on the row-major GEMM, and the oracle's; prompt portions and decoded tokens."""
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
    assert close(got[True], got[False], "bfloat16")
    assert close(got[True], oracle_logits("d", cfg, W, toks), "bfloat16")
    eng = engine(path, "cuda", "float32")
    assert rel(replay_all(eng, "f", toks, [30, 2, 9]), oracle_logits("d", cfg, W, toks)) < tol("float32")


def test_registry_and_config(tmp_path_factory):
    from vgate.models.config import HybridArch, resolve_arch
    from vgate.models.hybrid import tensor_shapes
    path, cfg, W = model_dir(tmp_path_factory, "a")
    a = resolve_arch(path)
    assert isinstance(a, HybridArch) and a.family == "livitar" and a.arrangement == "hyper_pre_norm" and a.streams == 3
    assert [L.kind for L in a.layers] == ["window_attention", "linear_attention", "window_attention", "linear_attention"]
    m0, m1, m2 = (a.layers[i].mixer for i in range(3))
    assert m0["dist_bias"] == {"kind": "table", "far": 21.0} and m0["q_temp"] == {"coef": 0.4, "every": 5} and m0["window"] is None
    assert m1["rot"]["layout"] == "half" and m1["k_scale"] == 10 ** -0.5 and m1["norm_weight"] is False
    assert m2["dist_bias"] == {"kind": "log"} and m2["head_temp"] and m2["gate"] == "sigmoid"
    assert a.layers[1].mlp is None and a.layers[3].mlp["router"]["score"] == "softmax" and "shared" not in a.layers[3].mlp
    open_shapes = tensor_shapes(a, nominal=None)
    assert open_shapes["l0.mix.rel"] == (None, 6) and open_shapes["l0.hc2.mix"] == (3, 3) and "l1.norm2" not in open_shapes
    assert set(open_shapes) == set(W)
    t = resolve_arch("livitar-tiny")
    assert t.family == "livitar" and t.num_params() > 0


# --------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("B,far", [(16, 200), (7, 21), (2, 3), (32, 256), (12, 60), (9, 100.5), (16, 1000), (8, 108)])
def test_distance_buckets(B, far):
    """The per-distance expansion of a bucket table: one row per distance below B // 2, log-spaced rows
    above, the last row for everything from ``far`` on."""
    from vgate.models.mixers import distance_buckets
    rows = distance_buckets(B, far)
    assert rows == [oracle.rel_bucket(n, B, far) for n in range(len(rows))]
    assert rows[-1] == B - 1 and all(oracle.rel_bucket(n, B, far) == B - 1 for n in (len(rows), 5 * len(rows), 10 ** 6))
    assert rows[: B // 2] == list(range(B // 2)) and all(b >= a for a, b in zip(rows, rows[1:]))


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


def _run_attention(d, dt, q, k, v, gate, H, G, scale, bias, tables, steps, temp=None, q_temp=(0.0, 1), unit=False,
                   transposed=False, prefill_kernel=0):
    """Feed sequences through window_write / window_attn (full causal, with a distance term) in the given
    steps (per-sequence new-token counts); returns each sequence's outputs [T, H * V]. ``transposed``: keep
    the transposed value copy, which selects the MFMA kernels (GPU, bf16)."""
    from vgate.models.mixers import WindowAttention
    from vgate.ops import seq
    S, D, V = len(q), q[0].shape[1] // H, v[0].shape[1] // G
    pages = int(max(max(t) for t in tables)) + 1
    kc = torch.full((pages, G, 16, D), 9.0, dtype=dt, device=d)
    vc = torch.full((pages, G, 16, V), -9.0, dtype=dt, device=d)
    vt = torch.full((pages, G, V, 16), -9.0, dtype=dt, device=d) if transposed else None
    bt = torch.zeros(S, max(len(t) for t in tables), dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, : len(t)] = torch.tensor(t, dtype=torch.int32)
    bt = bt.to(d)
    none = torch.zeros(0, device=d)
    ones = torch.ones(D, device=d) if unit else None
    kind, ba, bb = bias
    done = [0] * S
    outs = [[] for _ in range(S)]
    for new in steps:
        ctx = [done[s] + new[s] for s in range(S)]
        pos, slots, qs, cl = _step_meta(new, ctx, tables, d)
        cat = lambda xs: torch.cat([xs[s][done[s]: ctx[s]] for s in range(S)]).to(d, dt)  # noqa: E731
        T = int(qs[-1])
        qo = torch.zeros(T, H * D, dtype=dt, device=d)
        seq.window_write(cat(q), cat(k), cat(v), ones, ones, 1e-6, False, pos, slots, none, 0, None, kc, vc, qo, H, G, vt=vt,
                         q_head_scale=None if temp is None else temp.to(d), q_temp_coef=q_temp[0], q_temp_every=q_temp[1])
        o = torch.zeros(T, H * V, dtype=dt, device=d)
        seq.window_attn(qo, kc, vc, None, None, bt, cl, qs, o, scale, H, WindowAttention.FULL, 0, None, None, vt=vt,
                        prefill_kernel=prefill_kernel, bias_kind=kind, bias_a=ba.to(d), bias_b=None if bb is None else bb.to(d),
                        gate=None if gate is None else cat(gate))
        for s in range(S):
            outs[s].append(o[int(qs[s]): int(qs[s + 1])].float().cpu())
        done = ctx
    return [torch.cat(x) for x in outs]


def _want_attention(q, k, v, gate, H, G, scale, bias_fn, temp=None, q_temp=(0.0, 1), unit=False):
    """The oracle's causal attention of one sequence with bias_fn(head, distances [n, m]) added to the scores."""
    T, D, V = q.shape[0], q.shape[1] // H, v.shape[1] // G
    q3, k3, v3 = q.double().view(T, H, D), k.double().view(T, G, D), v.double().view(T, G, V)
    if unit:
        q3, k3 = oracle.unit_rms(q3, 1e-6), oracle.unit_rms(k3, 1e-6)
    pos = torch.arange(T)
    q3 = q3 * (1.0 + q_temp[0] * torch.log(torch.floor((pos + 1).double() / q_temp[1]) + 1.0))[:, None, None]
    dist = (pos[:, None] - pos[None, :]).clamp(min=0)
    out = torch.empty(T, H, V, dtype=torch.float64)
    for h in range(H):
        s = scale * (1.0 if temp is None else float(temp[h]))
        out[:, h] = oracle.attend(q3[:, h] * s, k3[:, h // (H // G)], v3[:, h // (H // G)], bias_fn(h, dist))
    out = out.reshape(T, H * V)
    return (out * torch.sigmoid(gate.double()) if gate is not None else out).float()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("kind", ["log", "table", "table_wide"])
def test_attention_distance_terms_on_crafted_keys(device, f32, kind):
    """The attention ops alone on crafted keys: for chosen query positions one key is made to dominate (it
    and the query are scaled along a probe direction): a key hundreds back, the first token, keys at page
    borders, keys at the distances where the table changes rows and where its last row begins (one before,
    at, one after). A distance that is one off moves the output by O(1), which the shifted oracle shows. Run
    as one prompt, as portions cut inside pages, and token by token over scattered, reused pages; FMA and
    both MFMA kernels; with the per-head and per-position temperatures and the output gate."""
    from vgate.models.mixers import distance_buckets
    from vgate.ops import seq
    dt = torch.float32 if f32 else torch.bfloat16
    g = torch.Generator().manual_seed(11)
    H, G, D, V, T = 4, 2, 8, 6, 310
    d = torch.device(device)
    q, k, v, gate = (torch.randn(T, n, generator=g) * 0.4 for n in (H * D, G * D, G * V, H * V))
    probe = torch.randn(D, generator=g)
    probe /= probe.norm()
    far = {"log": 0, "table": 40, "table_wide": 2500}[kind]   # (the wide table is read from global memory by the MFMA kernels)
    rows = 10
    queries = [309, 300, 290, 277, 260, 255, 200, 131, 64, 48]
    dists = [305, 300, far - 1, far, far + 1, 16, 33, 131, 0, 47] if kind == "table" else [305, 300, 1, 2, 250, 16, 33, 131, 0, 47]
    for n, (i, dd) in enumerate(zip(queries, dists)):
        j = i - dd
        k[j].view(G, D)[n % G] += 6.0 * probe
        q[i].view(H, D)[(n % G) * (H // G) + n % (H // G)] += 4.0 * probe
    q, k, v, gate = (x.to(dt).float() for x in (q, k, v, gate))
    temp = torch.tensor([0.7, 1.0, 1.6, 1.2])
    if kind == "log":
        r1, r2 = torch.tensor([0.9, 0.2, 1.4, 0.5]), torch.tensor([0.3, 2.0, 0.05, 1.0])
        bias = (seq.BIAS_LOG, r1, r2)
        fn = lambda h, dist, sh=0: -float(r1[h]) * torch.log(1.0 + float(r2[h]) * (dist + sh).double())  # noqa: E731
    else:
        relt = (2.0 * torch.randn(rows, H, generator=g)).to(torch.bfloat16).float()
        bias = (seq.BIAS_TABLE, relt[torch.tensor(distance_buckets(rows, far))].t().contiguous(), None)
        fn = lambda h, dist, sh=0: relt[:, h].double()[torch.tensor(  # noqa: E731
            [[oracle.rel_bucket(int(x) + sh, rows, far) for x in r] for r in dist.tolist()])]
    qt = (0.35, 16)
    want = _want_attention(q, k, v, gate, H, G, 0.5, fn, temp, qt)
    tables = [[7, 2, 9, 4, 11, 0, 5, 13, 1, 8, 3, 6, 10, 12, 14, 15, 16, 17, 18, 19]]
    for steps in ([[T]], [[61], [2], [35], [1], [1], [210]], [[T - 70]] + [[1]] * 70):
        for mfma in ([None, 0, 1] if device == "cuda" and not f32 else [None]):
            got = _run_attention(d, dt, [q], [k], [v], [gate], H, G, 0.5, bias, tables, steps, temp, qt,
                                 transposed=mfma is not None, prefill_kernel=mfma or 0)[0]
            assert rel(got, want) < (3e-5 if f32 else 2e-2), (len(steps), mfma)
    # the crafted keys matter: every distance taken one too large moves the answer
    assert rel(_want_attention(q, k, v, gate, H, G, 0.5, lambda h, dist: fn(h, dist, 1), temp, qt), want) > 0.02


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,V", [(2, 1, 8, 4), (8, 1, 16, 24), (2, 2, 160, 144)])
def test_attention_batch_and_page_reuse(device, H, G, D, V):
    """Two sequences in one step against each alone; the second takes over pages the first one used
    (stale keys and values in them must not be seen); unit-RMS queries and keys; eight query heads on one
    key / value head; heads wider than 128."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(12)
    d = torch.device(device)
    mk = lambda T: tuple(torch.randn(T, n, generator=g) for n in (H * D, G * D, G * V, H * V))  # noqa: E731
    (qa, ka, va, ga), (qb, kb, vb, gb) = mk(70), mk(37)
    r1, r2 = torch.linspace(0.6, 1.1, H), torch.linspace(0.5, 0.1, H)
    fn = lambda h, dist: -float(r1[h]) * torch.log(1.0 + float(r2[h]) * dist.double())  # noqa: E731
    bias = (seq.BIAS_LOG, r1, r2)
    wa, wb = (_want_attention(q, k, v, gg, H, G, 0.8, fn, unit=True) for q, k, v, gg in ((qa, ka, va, ga), (qb, kb, vb, gb)))
    got = _run_attention(d, torch.float32, [qa, qb], [ka, kb], [va, vb], [ga, gb], H, G, 0.8, bias,
                         [[3, 1, 4, 0, 2], [6, 5, 7]], [[30, 1], [2, 30], [38, 6]], unit=True)
    assert rel(got[0], wa) < 3e-5 and rel(got[1], wb) < 3e-5
    got = _run_attention(d, torch.float32, [qb], [kb], [vb], [gb], H, G, 0.8, bias, [[3, 1, 4]], [[20], [17]], unit=True)
    assert rel(got[0], wb) < 3e-5   # b again on a's pages, from position 0
    if device == "cuda":   # the MFMA kernels: rows of two sequences, of several tokens and of one
        for kern in (0, 1):
            got = _run_attention(d, torch.bfloat16, [qa, qb], [ka, kb], [va, vb], [ga, gb], H, G, 0.8, bias,
                                 [[3, 1, 4, 0, 2], [6, 5, 7]], [[30, 1], [2, 30], [38, 6]], unit=True, transposed=True,
                                 prefill_kernel=kern)
            assert rel(got[0], wa) < 2e-2 and rel(got[1], wb) < 2e-2, kern


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("every", [1, 4, 16])
def test_query_temperatures(device, every):
    """window_write's query multipliers: per head, and per position with steps of the floor at multiples of
    ``every`` minus one (positions just before, at and after them); keys are left alone."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(13)
    H, G, D, V, T = 3, 1, 6, 5, 9
    d = torch.device(device)
    q, k, v = (torch.randn(T, n, generator=g) for n in (H * D, G * D, G * V))
    pos = torch.tensor([0, every - 1, every, 2 * every - 2, 2 * every - 1, 2 * every, 1000, 1023, 5], dtype=torch.int32).clamp(min=0)
    slots = torch.tensor([3, 4, 5, 17, 18, 31, 6, 7, -1], dtype=torch.int32)
    temp = torch.tensor([0.5, 1.0, 2.5])
    kc, vc = torch.full((2, G, 16, D), 7.0, device=d), torch.full((2, G, 16, V), 7.0, device=d)
    qo = torch.zeros(T, H * D, device=d)
    seq.window_write(q.to(d), k.to(d), v.to(d), None, None, 1e-5, False, pos.to(d), slots.to(d), torch.zeros(0, device=d), 0, None,
                     kc, vc, qo, H, G, q_head_scale=temp.to(d), q_temp_coef=0.3, q_temp_every=every)
    grow = 1.0 + 0.3 * torch.log(torch.floor((pos + 1).double() / every) + 1.0)
    want = q.double().view(T, H, D) * temp.double()[None, :, None] * grow[:, None, None]
    assert rel(qo.cpu()[:-1], want.reshape(T, -1)[:-1]) < 1e-6
    assert rel(kc.cpu().view(32, D)[slots[:-1].long()], k[:-1]) < 1e-6
    assert float((kc == 7.0).sum()) == (32 - (T - 1)) * D   # the padding row wrote nothing


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,V,dims", [(2, 8, 8, 8), (3, 10, 6, 6), (1, 5, 9, 0), (2, 64, 32, 64), (1, 130, 16, 100)])
def test_retention_alone(device, H, D, V, dims):
    """linear_attn with half-split rotary positions, a key scale, a weightless head norm and a SiLU gate
    against the oracle's retention: one portion, cuts (also through the chunked scan), single tokens, a slot
    with garbage in it, positions in the hundreds."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(14)
    d = torch.device(device)
    W, T = 12, 330
    h = torch.randn(T, W, generator=g)
    m = {"heads": H, "dim": D, "vdim": V, "rot": {"base": 300.0, "dims": dims}, "decay": [0.5, 0.93, 0.999][:H]}
    t = {n: torch.randn(o, W, generator=g) / math.sqrt(W) for n, o in (("q", H * D), ("k", H * D), ("v", H * V), ("g", H * V))}
    t["o"] = torch.eye(H * V)
    want, _ = oracle.retention(h.double(), m, t, "", 1e-6)
    q, k, v, gg = (h @ t[n].T for n in ("q", "k", "v", "g"))
    inv = seq.rope_inv_freq(dims, 300.0, d) if dims else None
    dec = torch.tensor(m["decay"], dtype=torch.float32, device=d)
    for cuts in ([T], [1] * 20 + [260, 2, 48], [300, 30]):
        state = torch.full((3, H, D, V), 5.0, device=d)   # garbage: a portion at position 0 starts from zero
        out, at = [], 0
        for n in cuts:
            o = torch.zeros(n, H * V, device=d)
            i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=d)  # noqa: E731
            sl = lambda x: x[at: at + n].contiguous().to(d)  # noqa: E731
            seq.linear_attn(sl(q), sl(k), sl(v), sl(gg), None, dec, 1.0, 1.0, False, None, False, True, state, i32([1]),
                            i32([at + n]), i32([0, n]), o, 1e-6, k_scale=D ** -0.5, positions=i32(list(range(at, at + n))),
                            inv_freq=inv, rot_dims=dims, rot_half=True)
            out.append(o.cpu())
            at += n
        assert rel(torch.cat(out), want) < 1e-4, cuts
        assert float(state[0].min()) == 5.0 and float(state[2].max()) == 5.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S", [1, 2, 3, 5])
def test_stream_copies_and_tanh_norm(device, S):
    """hyper_mix (a sublayer's write to the copies, the next one's normed read, the copies' sum) and
    tanh_norm_rows against the oracle's formulas; the mix matrix is indexed [from, to]."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(15)
    d = torch.device(device)
    T, W = 7, 33
    xs = torch.randn(S, T, W, generator=g)
    y = torch.randn(T, W, generator=g)
    t = {"hc.in": torch.randn(S, generator=g), "hc.out": torch.randn(S, generator=g), "hc.mix": torch.randn(S, S, generator=g),
         "n": torch.randn(W, generator=g), "n.b": torch.randn(W, generator=g), "n.alpha": torch.tensor(0.7)}
    new = oracle.hyper_step(xs.double(), {k: v.double() for k, v in t.items()}, "hc.", lambda u: y.double(), lambda u: u)
    read = oracle.tanh_norm(torch.einsum("s,snw->nw", t["hc.in"].double(), new), t, "n")
    xd, h, sm = xs.clone().to(d), torch.zeros(T, W, device=d), torch.zeros(T, W, device=d)
    f = lambda x: x.to(d).float().contiguous()  # noqa: E731
    seq.hyper_mix(xd, y.to(d), f(t["hc.mix"]), f(t["hc.out"]), read_w=f(t["hc.in"]), alpha=f(t["n.alpha"].reshape(1)), w=f(t["n"]),
                  b=f(t["n.b"]), h_out=h, sum_out=sm)
    assert rel(xd, new) < 1e-6 and rel(h, read) < 1e-5 and rel(sm, new.sum(0)) < 1e-6
    if S > 1:   # [from, to], not its transpose
        assert rel(xd, torch.einsum("ts,snw->tnw", t["hc.mix"].double(), xs.double()) + t["hc.out"].double()[:, None, None] * y.double()) > 0.1
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=d)
    out = torch.zeros(3, W, device=d)
    seq.tanh_norm_rows(sm, f(t["n.alpha"].reshape(1)), f(t["n"]), f(t["n.b"]), out, rows=rows)
    assert rel(out, oracle.tanh_norm(new.sum(0)[rows.cpu().long()], t, "n")) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top", [(5, 2), (12, 3), (1, 1), (4, 4), (70, 5)])
def test_softmax_router(device, E, top):
    """moe_route with softmax scores over all experts, renormalised over the chosen and scaled; a shared
    row added by moe_combine."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(16)
    d = torch.device(device)
    T, W = 11, 6
    z = 3.0 * torch.randn(T, E, generator=g)
    idx, wts = torch.zeros(T, top, dtype=torch.int32, device=d), torch.zeros(T, top, device=d)
    seq.moe_route(z.to(d), None, top, 1e-20, idx, wts, softmax=True, scale=1.75)
    s = torch.softmax(z.double(), -1)
    ts, ti = torch.topk(s, top, -1)
    assert torch.equal(idx.cpu().long().sort(-1).values, ti.sort(-1).values)
    assert rel(wts.cpu().sum(-1), torch.full((T,), 1.75)) < 1e-6
    assert rel(wts.cpu(), torch.gather(s, 1, idx.cpu().long()) / ts.sum(-1, keepdim=True) * 1.75) < 1e-5
    y, add = torch.randn(T * top, W, generator=g), torch.randn(T, W, generator=g)
    pos = torch.randperm(T * top, generator=g).int()
    out = torch.zeros(T, W, device=d)
    seq.moe_combine(y.to(d), pos.to(d), wts, out, add=add.to(d))
    want = (y[pos.long()].view(T, top, W) * wts.cpu()[:, :, None]).sum(1) + add
    assert rel(out, want) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("K", [136, 64, 8, 520])
def test_large_row_major_gemm_forms(K):
    """The LDS-tiled form of the row-major GEMM (hundreds of rows, wide outputs) against the torch form: plain
    with a bias, a gated pair, grouped per expert with gathered rows (an empty group, groups that are not whole
    tiles), a k range that is not a whole number of k-steps, outputs that are not whole tiles."""
    from vgate.ops import seq
    g = torch.Generator().manual_seed(17)
    d = torch.device("cuda")
    T, top, E, N = 700, 2, 5, 520
    bf = lambda *s: (torch.randn(*s, generator=g) / math.sqrt(s[-1])).to(torch.bfloat16)  # noqa: E731
    a, w, w2, bias = torch.randn(T, K, generator=g).to(torch.bfloat16), bf(N, K), bf(N, K), torch.randn(N, generator=g)
    for kw in ({"bias": bias}, {"w2": w2, "act": seq.ACT_SILU_MUL}):
        cpu, gpu = torch.zeros(1100, N), torch.zeros(1100, N, device=d)
        big = torch.cat([a, a.flip(0)])[:1100].contiguous()
        seq.gemm(big, w, cpu, **kw)
        seq.gemm(big.to(d), w.to(d), gpu, **{k: (v.to(d) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()})
        assert rel(gpu, cpu) < 2e-5, list(kw)
    idx = torch.randint(0, E - 1, (T, top), generator=g).int()   # expert E - 1 gets no rows
    idx[:, 1] = (idx[:, 0] + 1 + torch.randint(0, E - 2, (T,), generator=g).int()) % (E - 1)
    rows, pos, off = (torch.zeros(n, dtype=torch.int32) for n in (T * top, T * top, E + 1))
    seq.moe_sort(idx, E, rows, pos, off)
    we, we2, wd = bf(E, N, K), bf(E, N, K), bf(E, K, N)
    for kw in ({}, {"w2": we2, "act": seq.ACT_SILU_MUL}):
        cpu, gpu = torch.zeros(T * top, N), torch.zeros(T * top, N, device=d)
        seq.gemm(a, we, cpu, a_rows=rows, group_off=off, **kw)
        seq.gemm(a.to(d), we.to(d), gpu, a_rows=rows.to(d), group_off=off.to(d),
                 **{k: (v.to(d) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()})
        assert rel(gpu, cpu) < 2e-5, list(kw)
    mid = torch.randn(T * top, N, generator=g).to(torch.bfloat16)
    cpu, gpu = torch.zeros(T * top, K), torch.zeros(T * top, K, device=d)
    seq.gemm(mid, wd, cpu, group_off=off)
    seq.gemm(mid.to(d), wd.to(d), gpu, group_off=off.to(d))
    assert rel(gpu, cpu) < 2e-5   # (K columns out: below the wide form's range unless K >= 512; both paths are right)
