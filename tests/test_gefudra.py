"""Gefudra (pre-norm layers with a residual multiplier, a stretch of layers that runs several times with the
same weights behind an input matrix, latent attention over a sliding window with a sink, two-map attention with
softcap and half-split rotation, a shifted decayed recurrence with a bonus, clamped dense feed-forward, tied
and scaled logits) in the engine, against the plain implementation of tests/gefudra_oracle.py.

Small configurations with random weights are written to a temporary folder (config.json +
model.safetensors) and run through ``LLMEngine.replay_step`` / ``add_request`` on the CPU device
(unfused torch forms of the ops) and, marked ``gpu``, on the HIP kernels, in fp32 and bf16.
"""
from __future__ import annotations

import json
import math

import pytest
import torch

import gefudra_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


# ------------------------------------------------------------------------------------ configurations
def _ff(n, limit=1.5):
    return {"kind": "dense", "ff": n, "limit": limit}


def _lat(H, D, V, kv, qr, win, mlp, scale=None):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": H, "dim": D, "vdim": V, "kv_rank": kv, "q_rank": qr, "scale": scale or 2.0 / math.sqrt(D),
                      "mask": {"size": win}}}


def _att(H, G, D, V, dims, base, cap, diff, mlp, scale=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale or 2.0 / math.sqrt(D),
                      "rot": {"base": base, "dims": dims}, "softcap": cap, "diff": diff}}


def _wkv(H, D, mlp):
    return {"type": "wkv", "mlp": mlp, "mixer": {"heads": H, "dim": D}}


def _model(width, vocab, layers, loop, mult, scale, eps=1e-5):
    cfg = {"architecture": "Gefudra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult,
           "logit_scale": scale, "layers": layers}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def config_a():
    """Unequal everything: sizes that are no multiple of 8 (the fp32-FMA attention kernels in bf16 too), key size
    != value size, fewer rotated dims than the head, grouped key/value heads, a window shorter than a page, a
    strong softcap, layers without feed-forward, the loop over the middle, a vocabulary that is no multiple of 4."""
    return _model(40, 50, [
        _att(4, 2, 6, 10, 4, 100.0, 2.0, 0.3, _ff(24)),
        _lat(3, 10, 6, 12, 7, 5, None),
        _wkv(2, 5, None),
        _lat(2, 6, 9, 20, 11, 19, _ff(16, 0.4)),
        _wkv(3, 12, _ff(24))], (1, 4, 2), 0.4, 1.7)


def config_b():
    """Values that are 1 or equal: one head everywhere, a window of one token, a loop over all layers that runs
    once, multipliers of exactly 1, every dim rotated."""
    return _model(24, 32, [
        _wkv(1, 4, _ff(8)),
        _lat(1, 4, 4, 4, 4, 1, _ff(8)),
        _att(1, 1, 4, 4, 4, 10.0, 30.0, 0.5, None)], (0, 3, 1), 1.0, 1.0, eps=1e-6)


def config_c():
    """Page-scale geometry on the MFMA kernels' sizes: windows that end inside the third page, exactly at a page
    border and one past it, three passes through the loop, the loop at the end, no loop input before layer 0."""
    return _model(64, 96, [
        _lat(4, 16, 32, 32, 24, 37, _ff(48)),
        _att(4, 2, 16, 32, 8, 10000.0, 25.0, 0.7, _ff(48)),
        _wkv(2, 16, None),
        _lat(2, 32, 16, 48, 16, 16, _ff(48)),
        _att(2, 2, 32, 16, 32, 500.0, 5.0, 0.2, None),
        _lat(4, 8, 8, 16, 8, 17, None)], (3, 6, 3), 0.35, 1.5, eps=1e-6)


def config_d():
    """Sizes in the range the fragment-packed MFMA GEMMs take (width 512, projections in multiples of 64); no loop."""
    return _model(512, 704, [
        _lat(4, 64, 64, 128, 192, 33, _ff(1024, 4.0)),
        _att(8, 2, 64, 64, 64, 10000.0, 20.0, 0.4, _ff(1024, 4.0)),
        _wkv(4, 64, _ff(1024, 4.0))], None, 0.5, 1.0, eps=1e-6)


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d}


def make_tensors(cfg: dict, seed: int) -> dict:
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.5):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    def unit(n):
        return torch.rand(n, generator=g).to(torch.bfloat16)

    t = {"embed": torch.randn(V, W, generator=g).to(torch.bfloat16), "final.norm": vec(W, 1.0, 0.3)}
    if cfg.get("loop"):
        t["loop.in"] = (torch.cat([torch.eye(W), 0.5 * torch.eye(W)], 1) + 0.5 * torch.randn(W, 2 * W, generator=g) / math.sqrt(W)
                        ).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        p, m, x = f"l{i}.", L["mixer"], f"l{i}.mix."
        t[p + "norm1"] = vec(W, 1.0, 0.3)
        H, D = m["heads"], m["dim"]
        if L["type"] == "latent_attention":
            Vd, kr, qr = m["vdim"], m["kv_rank"], m["q_rank"]
            t.update({x + "dq": mat(qr, W), x + "dq.norm": vec(qr, 1.0, 0.3), x + "uq": mat(H * D, qr, 2.0),
                      x + "dkv": mat(kr, W), x + "dkv.norm": vec(kr, 1.0, 0.3), x + "uk": mat(H * D, kr, 2.0),
                      x + "uv": mat(H * Vd, kr), x + "sink": vec(H, 0.5, 1.0), x + "g": mat(H * Vd, W, 2.0), x + "o": mat(W, H * Vd)})
        elif L["type"] == "attention":
            Vd, G = m["vdim"], m["kv_heads"]
            t.update({x + "q": mat(H * 2 * D, W, 2.0), x + "k": mat(G * 2 * D, W, 2.0), x + "v": mat(G * Vd, W),
                      x + "g": mat(H * Vd, W, 2.0), x + "o": mat(W, H * Vd)})
            t.update({x + n: vec(D, 0.0, 0.6 / math.sqrt(D)) for n in ("lq1", "lk1", "lq2", "lk2")})
        else:
            n = H * D
            low = 3 + i
            t.update({x + "mu." + s: unit(W) for s in "rkvgw"})
            t.update({x + "r": mat(n, W), x + "k": mat(n, W), x + "v": mat(n, W), x + "g": mat(n, W, 2.0), x + "w1": mat(low, W),
                      x + "w2": mat(n, low, 2.0), x + "w0": vec(n, -1.5, 1.0), x + "u": vec(n, 0.5, 0.5).view(H, D),
                      x + "norm": vec(n, 1.0, 0.3), x + "o": mat(W, n)})
        if L.get("mlp"):
            f = L["mlp"]["ff"]
            t.update({p + "norm2": vec(W, 1.0, 0.3), p + "mlp.gate": mat(f, W, 2.0), p + "mlp.up": mat(f, W, 2.0),
                      p + "mlp.down": mat(W, f)})
    return t


_MODELS: dict = {}


def model_dir(tmp_path_factory, name: str):
    """(folder, config dict, tensors) of a named test model, written once per session."""
    if name not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]()
        t = make_tensors(cfg, seed={"a": 3, "b": 5, "c": 7, "d": 9}[name])
        d = tmp_path_factory.mktemp("gefudra_" + name)
        save_file({k: v.contiguous() for k, v in t.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[name] = (str(d), cfg, t)
    return _MODELS[name]


_ORACLE: dict = {}


def oracle_run(name, cfg, W, tokens):
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        lg, streams = oracle.forward(cfg, W, list(tokens))
        _ORACLE[key] = (lg.float(), streams.float())
    return _ORACLE[key]


def oracle_logits(name, cfg, W, tokens):
    return oracle_run(name, cfg, W, tokens)[0]


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
    """fp32: the whole result within tol. bf16: per token, the median within tol and nine in ten within 0.15 (a
    fault of a mechanism moves most tokens by O(1))."""
    if dtype == "float32":
        return rel(got, want) < tol(dtype)
    g, w = got.double().cpu(), want.double().cpu()
    e = (g - w).pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
    return float(e.median()) < tol(dtype) and float((e < 0.15).double().mean()) >= 0.9


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
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_layers_match_oracle(tmp_path_factory, device, name):
    """The stream after every layer run; a looped layer counts once per pass."""
    path, cfg, W = model_dir(tmp_path_factory, name)
    toks = tokens_of(cfg, 23, seed=2)
    eng = engine(path, device, "float32")
    eng.model.capture_layers = []
    replay_all(eng, "l", toks, [len(toks)])
    want = oracle_run(name, cfg, W, toks)[1]
    lp = cfg["loop"]
    runs = len(cfg["layers"]) + (lp["stop"] - lp["start"]) * (lp["times"] - 1)
    assert len(eng.model.capture_layers) == want.shape[0] == runs
    for i, got in enumerate(eng.model.capture_layers):
        assert rel(got[: len(toks)], want[i]) < 1e-4, f"stream after layer run {i}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[1], [30], [2, 2, 2, 3, 5, 7, 16, 17], [15, 1, 16, 2, 14], [47, 2]])
def test_portions_and_decoding_match_whole(tmp_path_factory, device, dtype, cuts):
    """Prefill against token-by-token decoding and portions of several sizes down to two tokens (cuts inside
    pages and at their borders, inside and at the ends of the windows); the tail decodes one token at a time."""
    path, cfg, W = model_dir(tmp_path_factory, "c")
    toks = tokens_of(cfg, 120, seed=3)
    eng = engine(path, device, dtype)
    whole = replay_all(eng, "whole", toks, [len(toks)])
    cut = replay_all(eng, "cut", toks, cuts)
    assert rel(cut, whole) < 2e-5 if dtype == "float32" else close(cut, whole, dtype)
    assert close(cut, oracle_logits("c", cfg, W, toks), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_portion_through_the_chunked_scan(tmp_path_factory, device):
    """A portion of several hundred tokens (the recurrence's chunked form on the GPU) and then single tokens."""
    path, cfg, W = model_dir(tmp_path_factory, "c")
    toks = tokens_of(cfg, 420, seed=6)
    eng = engine(path, device, "float32", pages=28)
    got = replay_all(eng, "p", toks, [300, 90, 2])
    want = oracle_logits("c", cfg, W, toks)
    assert rel(got, want) < tol("float32") and rel(got[-20:], want[-20:]) < tol("float32")


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
    assert isinstance(a, HybridArch) and a.family == "gefudra" and a.arrangement == "pre_norm"
    assert a.loop == (1, 4, 2) and a.residual_mult == 0.4 and a.logit_scale == 1.7 and a.tie_embeddings
    assert [i for i, _ in a.run_order()] == [0, 1, 2, 3, 1, 2, 3, 4]
    assert [f for _, f in a.run_order()] == [False, True, False, False, True, False, False, False]
    assert [L.kind for L in a.layers] == ["window_attention", "latent_attention", "wkv", "latent_attention", "wkv"]
    m0, m1 = a.layers[0].mixer, a.layers[1].mixer
    assert m0["maps"] == {"count": 2, "init": 0.3} and m0["softcap"] == 2.0 and m0["rot"] == {"dims": 4, "base": 100.0, "layout": "half"}
    assert m0["window"] is None and m0["gate"] == "sigmoid"
    assert m1["window"] == 5 and m1["sink"] and m1["rot_dim"] == 0
    assert a.layers[1].mlp is None and a.layers[3].mlp == {"kind": "dense", "ff": 16, "act": "clamped", "limit": 0.4}
    open_shapes = tensor_shapes(a, nominal=None)
    assert open_shapes["l2.mix.w1"] == (None, 40) and open_shapes["loop.in"] == (40, 80) and "head" not in open_shapes
    assert open_shapes["l0.mix.q"] == (4 * 2 * 6, 40) and open_shapes["l0.mix.k"] == (2 * 2 * 6, 40)
    assert set(open_shapes) == set(W)
    b = resolve_arch(model_dir(tmp_path_factory, "b")[0])
    assert b.loop == (0, 3, 1) and [f for _, f in b.run_order()] == [True, False, False]
    t = resolve_arch("gefudra-tiny")
    assert t.family == "gefudra" and t.num_params() > 0


@pytest.mark.parametrize("device", DEVICES)
def test_preset_runs(device):
    eng = engine("gefudra-tiny", device, "bfloat16")
    lg = eng.replay_step([("x", list(range(20)), [0, 19])], ["x"])
    assert lg.shape == (2, 300) and bool(torch.isfinite(lg).all())


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


def _block_tables(tables, d):
    bt = torch.zeros(len(tables), max(len(t) for t in tables), dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, : len(t)] = torch.tensor(t, dtype=torch.int32)
    return bt.to(d)


STEPS_310 = ([[310]], [[61], [2], [35], [1], [1], [210]], [[240]] + [[1]] * 70)
SCATTERED = [[7, 2, 9, 4, 11, 0, 5, 13, 1, 8, 3, 6, 10, 12, 14, 15, 16, 17, 18, 19]]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("rank,window", [(16, 37), (12, 16), (24, 1), (16, 1 << 30)])
def test_latent_window_and_sink_on_crafted_keys(device, f32, rank, window):
    """The latent attention ops alone: for chosen query positions one cached row is made to dominate (it and the
    query are scaled along a probe direction): the oldest key inside the window, the first one outside it, the
    token itself, keys at page borders, the first token of the sequence, and for the unbounded window a key
    hundreds back. A window that is one off moves the output by O(1), which the shifted reference shows. One
    prompt, portions cut inside pages, and token by token over scattered pages; FMA and (rank a multiple of 8,
    bf16, GPU) MFMA kernels; the sink made comparable to the scores."""
    from vgate.ops import seq
    dt = torch.float32 if f32 else torch.bfloat16
    d = torch.device(device)
    g = torch.Generator().manual_seed(5)
    H, T, scale, eps = 3, 310, 0.7, 1e-5
    kv = torch.randn(T, rank, generator=g)
    w = (1.0 + 0.2 * torch.randn(rank, generator=g))
    qa = torch.randn(T, H, rank, generator=g) * 0.5
    sink = torch.tensor([1.5, -0.5, 3.0])
    probe = torch.randn(rank, generator=g)
    probe /= probe.norm()
    full = window >= T
    queries = [309, 300, 290, 277, 260, 255, 200, 131, 64, 48, 47]
    dists = [305, 300, 1, 2, 250, 16, 33, 131, 0, 47, 47] if full else \
        [window - 1, window, 0, window - 1, window, min(window - 1, 16), window + 15, window - 1, 0, window, window - 1]
    boosted = torch.zeros(T, dtype=torch.bool)
    for n, (i, dd) in enumerate(zip(queries, dists)):
        j = i - dd
        if j < 0 or boosted[j]:
            continue
        boosted[j] = True
        kv[j] = kv[j] * 0.3 + 4.0 * probe * math.sqrt(rank)   # survives the norm: the row points along the probe
        qa[i, n % H] += 5.0 * probe
    kv, qa = kv.to(dt).float(), qa.to(dt).float()

    def want_for(win, with_sink=True):
        c = oracle.rms(kv.double(), eps, w)
        c = c.to(dt).double() if not f32 else c
        out = torch.zeros(T, H, rank, dtype=torch.float64)
        for i in range(T):
            lo = max(0, i - win + 1)
            for h in range(H):
                p = oracle.sink_softmax((c[lo:i + 1] @ qa[i, h].double()) * scale, float(sink[h]) if with_sink else None)
                out[i, h] = p @ c[lo:i + 1]
        return out.float()

    want = want_for(window)
    for steps in STEPS_310:
        for mfma in ([False, True] if device == "cuda" and not f32 and rank % 8 == 0 else [False]):
            cache = torch.full((20, 16, rank), 7.0, dtype=dt, device=d)
            cache_t = torch.full((20, rank, 16), 7.0, dtype=dt, device=d) if mfma else None
            bt = _block_tables(SCATTERED, d)
            done, outs = 0, []
            for (n,) in steps:
                pos, slots, qs, cl = _step_meta([n], [done + n], SCATTERED, d)
                seq.latent_write(kv[done: done + n].to(d, dt), w.to(d), eps, pos, slots, torch.zeros(0, device=d), 0, cache, rank,
                                 cache_t=cache_t)
                ol = torch.zeros(n, H, rank, dtype=dt, device=d)
                seq.latent_attn(qa[done: done + n].to(d, dt).contiguous(), cache, bt, cl, qs, ol, scale, H, rank, 0,
                                cache_t=cache_t, window=window, sink=sink.to(d))
                outs.append(ol.float().cpu())
                done += n
            assert rel(torch.cat(outs), want) < (3e-5 if f32 else 2e-2), (len(steps), mfma)
    # the crafted keys matter: a window one token longer or shorter, or no sink, moves the answer
    assert rel(want_for(window, with_sink=False), want) > 0.02
    if not full:
        assert rel(want_for(window + 1), want) > 0.02
    if window > 1 and not full:
        assert rel(want_for(window - 1), want) > 0.02


def _two_map_reference(q, k, v, gate, H, G, D, V, scale, dims, base, cap, lam, out_scale, eps):
    """float64: two maps per head over shared values, combined, normed, gated (one sequence)."""
    T = q.shape[0]
    pos = torch.arange(T)
    q4 = oracle.turn_halves(q.double().view(T, H, 2, D), pos, dims, base)
    k4 = oracle.turn_halves(k.double().view(T, G, 2, D), pos, dims, base)
    v3 = v.double().view(T, G, V)
    out = torch.zeros(T, H, V, dtype=torch.float64)
    for i in range(T):
        for h in range(H):
            gq = h // (H // G)
            a = []
            for mp in range(2):
                s = (k4[: i + 1, gq, mp] @ q4[i, h, mp]) * scale
                if cap > 0:
                    s = cap * torch.tanh(s / cap)
                a.append(oracle.sink_softmax(s, None) @ v3[: i + 1, gq])
            out[i, h] = oracle.rms(a[0] - lam * a[1], eps) * out_scale
    return (out.reshape(T, H * V) * torch.sigmoid(gate.double())).float()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("H,G,D,V,dims,cap", [(4, 2, 8, 6, 4, 3.0), (2, 2, 16, 16, 16, 0.0), (3, 1, 6, 5, 6, 40.0)])
def test_two_map_attention_on_crafted_keys(device, f32, H, G, D, V, dims, cap):
    """The two-map attention ops alone (half-split rotation of the leading dims of every map, softcap, key heads
    2g + m sharing value head g, the maps' combination): a key hundreds back, the first token and keys at page
    borders are made dominant in one map or the other. One prompt, portions, and decoding over scattered pages;
    FMA and (bf16, GPU, key size a multiple of 8) both MFMA kernels."""
    from vgate.models.mixers import WindowAttention
    from vgate.ops import seq
    dt = torch.float32 if f32 else torch.bfloat16
    d = torch.device(device)
    g = torch.Generator().manual_seed(13)
    T, scale, base, lam, out_scale, eps = 310, 0.6, 50.0, 0.45, 0.7, 1e-5
    rep = H // G
    q, k, v, gate = (torch.randn(T, n, generator=g) * 0.4 for n in (H * 2 * D, G * 2 * D, G * V, H * V))
    probe = torch.zeros(D)
    probe[dims:] = 1.0            # unrotated entries keep the probe's direction at every position
    if dims == D:
        probe[:] = 0.0
    queries, dists = [309, 300, 290, 255, 200, 131, 64, 48], [305, 300, 1, 16, 33, 131, 0, 47]
    for n, (i, dd) in enumerate(zip(queries, dists)):
        j, h, mp = i - dd, n % H, n % 2
        if dims < D:
            k[j].view(G, 2, D)[h // rep, mp] += 6.0 * probe
            q[i].view(H, 2, D)[h, mp] += 4.0 * probe
        else:     # every entry turns: scale a random pair instead; the rotation must then be right for it to dominate
            k[j].view(G, 2, D)[h // rep, mp] *= 6.0
            q[i].view(H, 2, D)[h, mp] *= 4.0
    q, k, v, gate = (x.to(dt).float() for x in (q, k, v, gate))
    want = _two_map_reference(q, k, v, gate, H, G, D, V, scale, dims, base, cap, lam, out_scale, eps)
    # query rows regrouped (key/value head, map, head in group), as the mixer does at load
    qg = q.view(T, G, rep, 2, D).transpose(2, 3).reshape(T, H * 2 * D)
    inv_freq = seq.rope_inv_freq(dims, base, d)
    for steps in STEPS_310:
        for mfma in ([None, 0, 1] if device == "cuda" and not f32 and D % 8 == 0 else [None]):
            kc = torch.full((20, 2 * G, 16, D), 9.0, dtype=dt, device=d)
            vc = torch.full((20, G, 16, V), -9.0, dtype=dt, device=d)
            vt = torch.full((20, G, V, 16), -9.0, dtype=dt, device=d) if mfma is not None else None
            bt = _block_tables(SCATTERED, d)
            done, outs = 0, []
            for (n,) in steps:
                pos, slots, qs, cl = _step_meta([n], [done + n], SCATTERED, d)
                cut = lambda x: x[done: done + n].to(d, dt).contiguous()  # noqa: E731
                qo = torch.zeros(n, 2 * H * D, dtype=dt, device=d)
                seq.window_write(cut(qg), cut(k), cut(v), None, None, eps, False, pos, slots, inv_freq, dims, None, kc, vc, qo,
                                 2 * H, 2 * G, vt=vt, rot_half=True)
                both = torch.zeros(n, 2 * H * V, dtype=dt, device=d)
                seq.window_attn(qo, kc, vc, None, None, bt, cl, qs, both, scale, 2 * H, WindowAttention.FULL, 0, None, None, vt=vt,
                                prefill_kernel=mfma or 0, softcap=cap)
                o = torch.zeros(n, H * V, dtype=dt, device=d)
                seq.map_pair_combine(both, lam, out_scale, eps, cut(gate), o, H, G, V)
                outs.append(o.float().cpu())
                done += n
            assert rel(torch.cat(outs), want) < (5e-5 if f32 else 3e-2), (len(steps), mfma)
    # sensitivity: the other layout of the rotation, no softcap, or the maps swapped give another answer
    if cap > 0 and cap < 10:
        assert rel(_two_map_reference(q, k, v, gate, H, G, D, V, scale, dims, base, 0.0, lam, out_scale, eps), want) > 0.02
    assert rel(_two_map_reference(q, k, v, gate, H, G, D, V, scale, dims, base, cap, -lam, out_scale, eps), want) > 0.02


def _shifted_recurrence_reference(h, mu, Wr, Wk, Wv, Wg, z_of, u, nw, H, D, eps):
    """float64, token by token: the blends, the decays, the state read before its update with the bonus."""
    n, W = h.shape
    hd = h.double()
    prev = torch.cat([torch.zeros(1, W, dtype=torch.float64), hd[:-1]])
    x = [hd + (prev - hd) * mu[s].double() for s in range(5)]
    r, k, v = ((x[i] @ M.double().t()).view(n, H, D) for i, M in enumerate((Wr, Wk, Wv)))
    gate = torch.nn.functional.silu(x[3] @ Wg.double().t())
    w = torch.exp(-torch.exp(z_of(x[4]))).view(n, H, D)
    S = torch.zeros(H, D, D, dtype=torch.float64)
    out = torch.zeros(n, H, D, dtype=torch.float64)
    for i in range(n):
        kv = k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", S + u.double()[:, :, None] * kv, r[i])
        S = w[i][:, :, None] * S + kv
    return (oracle.rms(out, eps).reshape(n, H * D) * nw.double() * gate).float()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D", [(2, 5), (1, 16), (3, 40), (1, 130)])
def test_shifted_recurrence_alone(device, H, D):
    """shift_mix + the recurrence ops in fp32 against the token-by-token reference: two sequences of unequal
    length in portions (one of them several hundred tokens in one step: the chunked scan), single tokens, slots
    that hold another sequence's state and last row before they are taken again."""
    from vgate.ops import seq
    d = torch.device(device)
    g = torch.Generator().manual_seed(17 + D)
    W, eps, n = 24, 1e-5, H * D
    lens = [330, 41]
    mu = torch.rand(5, W, generator=g)
    Wr, Wk, Wv, Wg = (torch.randn(n, W, generator=g) / math.sqrt(W) for _ in range(4))
    Wz = torch.randn(n, W, generator=g) / math.sqrt(W)
    w0 = -2.0 + torch.randn(n, generator=g)
    u, nw = torch.randn(H, D, generator=g), 1.0 + 0.3 * torch.randn(n, generator=g)
    hs = [torch.randn(L, W, generator=g) for L in lens]
    z_of = lambda x: x @ Wz.double().t() + w0.double()  # noqa: E731
    want = [_shifted_recurrence_reference(h, mu, Wr, Wk, Wv, Wg, z_of, u, nw, H, D, eps) for h in hs]
    state = torch.randn(3, H, D, D, generator=g).to(d)    # garbage of earlier owners
    last = torch.randn(3, W, generator=g).to(d)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=d)
    done, outs = [0, 0], [[], []]
    for new in ([300, 7], [2, 1], [1, 30], [27, 3]):
        ctx = [done[s] + new[s] for s in range(2)]
        qs = torch.tensor([0, new[0], new[0] + new[1]], dtype=torch.int32, device=d)
        cl = torch.tensor(ctx, dtype=torch.int32, device=d)
        h = torch.cat([hs[s][done[s]: ctx[s]] for s in range(2)]).to(d)
        T = h.shape[0]
        x = torch.zeros(5, T, W, device=d)
        seq.shift_mix(h, last, mu.to(d), slots, cl, qs, x)
        r, k, v, gg = (x[i] @ M.to(d).t() for i, M in enumerate((Wr, Wk, Wv, Wg)))
        z = (x[4] @ Wz.to(d).t() + w0.to(d)).contiguous()
        out = torch.zeros(T, n, device=d)
        seq.linear_attn(r.contiguous(), k.contiguous(), v.contiguous(), gg.contiguous(), z, None, 1.0, 1.0, False, nw.to(d), False,
                        True, state, slots, cl, qs, out, eps, decay_exp=True, bonus=u.to(d).contiguous(), norm_full=True)
        outs[0].append(out[: new[0]].cpu())
        outs[1].append(out[new[0]:].cpu())
        done = ctx
    for s in range(2):
        assert rel(torch.cat(outs[s]), want[s]) < 2e-4, s
    assert rel(last[2].cpu(), hs[0][-1]) < 1e-6 and rel(last[0].cpu(), hs[1][-1]) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("f32", [True, False])
def test_residual_norm_pair_rows_and_clamped_pair(device, f32):
    """x += m y with the next norm; two row sets side by side; the clamped gated pair as a GEMM epilogue and as a
    row kernel, against the formulas."""
    from vgate.ops import seq
    dt = torch.float32 if f32 else torch.bfloat16
    d = torch.device(device)
    g = torch.Generator().manual_seed(23)
    for T, W in ((5, 40), (3, 4100)):
        x, y, w = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g).to(dt), 1.0 + 0.2 * torch.randn(W, generator=g)
        want_x = x.double() + 0.3 * y.double()
        xd, hd = x.clone().to(d), torch.zeros(T, W, dtype=dt, device=d)
        seq.residual_norm(xd, y.to(d), 0.3, w.to(d), 1e-5, hd)
        assert rel(xd.cpu(), want_x) < 1e-6
        assert rel(hd.float().cpu(), oracle.rms(want_x, 1e-5, w)) < (1e-6 if f32 else 4e-3)
        x2 = x.clone().to(d)
        seq.residual_norm(x2, y.to(d), -1.0)
        assert rel(x2.cpu(), x.double() - y.double()) < 1e-6
        pr = torch.zeros(T, 2 * W, dtype=dt, device=d)
        seq.pair_rows(x.to(d), x2, pr)
        assert rel(pr.float().cpu(), torch.cat([x, x2.cpu()], -1)) < (1e-7 if f32 else 4e-3)
    M, K, N, L = 9, 24, 16, 0.8
    a, wg, wu = (torch.randn(s, generator=g).to(dt) for s in ((M, K), (N, K), (N, K)))
    gf, uf = a.double() @ wg.double().t(), a.double() @ wu.double().t()
    gc = gf.clamp(max=L)
    want = gc * torch.sigmoid(1.702 * gc) * (uf.clamp(-L, L) + 1.0)
    out = torch.zeros(M, N, dtype=dt, device=d)
    seq.gemm(a.to(d), wg.to(d), out, w2=wu.to(d), act=seq.ACT_CLAMPED_GLU, limit=L, alpha=1.702)
    assert rel(out.float().cpu(), want) < (1e-5 if f32 else 1e-2)
    if not f32:
        gu = torch.cat([gf, uf], -1).to(dt)
        gc = gu[:, :N].double().clamp(max=L)
        want = gc * torch.sigmoid(1.702 * gc) * (gu[:, N:].double().clamp(-L, L) + 1.0)
        out = torch.zeros(M, N, dtype=dt, device=d)
        seq.glu_rows(gu.to(d), out, seq.ACT_CLAMPED_GLU, limit=L, alpha=1.702)
        assert rel(out.float().cpu(), want) < 1e-2
