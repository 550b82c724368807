"""Prefill and decode throughput of a layered hybrid design (Zadirax, Pozalorn, Livitar, Gefudra) beside the closest
transformer family, or beside another of the designs, at equal layer sizes (random weights, the same number
of layers), through the engine's own step path.

    python bench.py --design-compare [--design zadirax|pozalorn|livitar|gefudra] [--design-beside transformer|<design>]
                    [--design-sizes 1024,1536] [--design-prefill 2048] [--design-batch 32] [--design-context 512]

Both models run teacher-forced steps (``LLMEngine.replay_step``: cache manager, step metadata, model
forward and kernels; eager launches, nothing sampled):
  prefill: one request's prompt of ``--design-prefill`` tokens in one step            -> tokens/s
  decode : ``--design-batch`` requests with ``--design-context`` cached tokens each,
           one token per request and step                                             -> tokens/s
Prints one JSON line per (size, model) and a final summary line with the ratios.
"""
from __future__ import annotations

import json
import statistics
import time


def _engine(model: str, overrides: dict | None, tokens: int, seqs: int):
    from vgate.runtime.engine import EngineConfig, LLMEngine
    pages = (tokens + 15) // 16 + seqs
    return LLMEngine(EngineConfig(model=model, device="cuda:0", max_model_len=tokens + 16, max_num_seqs=seqs,
                                  max_num_batched_tokens=max(tokens, seqs) + 16, num_kv_blocks=pages,
                                  enable_prefix_caching=False, enforce_eager=True, warmup=False, prefill_autotune=False,
                                  async_scheduling=False, arch_overrides=overrides))


def _timed(fn, sync, reps: int) -> float:
    ts = []
    for _ in range(reps):
        sync()
        t0 = time.perf_counter()
        fn()
        sync()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts)


def measure(model: str, overrides: dict | None, prefill: int, batch: int, context: int, vocab: int) -> dict:
    import torch
    sync = torch.cuda.synchronize
    g = torch.Generator().manual_seed(1)
    out = {}
    # prefill: a fresh request each repetition (pages and slot are given back at its end)
    eng = _engine(model, overrides, prefill, 1)
    toks = torch.randint(0, vocab, (prefill,), generator=g).tolist()
    n = [0]

    def one_prefill():
        n[0] += 1
        eng.replay_step([(f"p{n[0]}", toks, [prefill - 1])], [f"p{n[0]}"])
    one_prefill()  # first launch of every kernel
    out["prefill_tok_s"] = round(prefill / _timed(one_prefill, sync, 5), 1)
    out["weights_gb"] = round(eng.model.weight_bytes() / 1e9, 3)
    del eng
    torch.cuda.empty_cache()
    # decode
    eng = _engine(model, overrides, batch * (context + 64), batch)
    ctx = [torch.randint(0, vocab, (context,), generator=g).tolist() for _ in range(batch)]
    for i in range(batch):
        eng.replay_step([(f"d{i}", ctx[i], [])], [])
    step = [0]

    def one_decode():
        step[0] += 1
        eng.replay_step([(f"d{i}", [(7 * i + step[0]) % vocab], [0]) for i in range(batch)], [])
    one_decode()
    out["decode_tok_s"] = round(batch / _timed(one_decode, sync, 20), 1)
    del eng
    torch.cuda.empty_cache()
    return out


# transformer overrides at equal width / heads / feed-forward / vocabulary
_QWEN = {1024: dict(hidden_size=1024, num_heads=8, num_kv_heads=2, intermediate_size=4096, vocab_size=32000, tie_embeddings=False),
         1536: dict(hidden_size=1536, num_heads=12, num_kv_heads=2, intermediate_size=8960, vocab_size=32000, tie_embeddings=False)}
# design -> (layers of its bench presets, "<design>-bench-<width>")
DESIGNS = {"zadirax": 4, "pozalorn": 3, "livitar": 3, "gefudra": 3}


def main(sizes: list[int], prefill: int = 2048, batch: int = 32, context: int = 512, design: str = "zadirax",
         only_design: bool = False, beside: str = "transformer") -> dict:
    layers = DESIGNS[design]
    if beside != "transformer" and DESIGNS.get(beside) != layers:
        raise ValueError(f"--design-beside {beside}: a design whose bench presets have {layers} layers, or transformer")
    summary = {}
    for w in sizes:
        preset = f"{design}-bench-{w}"
        a = measure(preset, None, prefill, batch, context, 32000)
        print(json.dumps({"width": w, "model": preset, **a}), flush=True)
        if only_design:
            continue
        if beside == "transformer":
            b = measure("qwen2.5-1.5b", dict(_QWEN[w], num_layers=layers), prefill, batch, context, 32000)
            print(json.dumps({"width": w, "model": f"qwen2 ({layers} layers, equal width)", **b}), flush=True)
        else:
            b = measure(f"{beside}-bench-{w}", None, prefill, batch, context, 32000)
            print(json.dumps({"width": w, "model": f"{beside}-bench-{w}", **b}), flush=True)
        summary[str(w)] = {"prefill_ratio": round(a["prefill_tok_s"] / b["prefill_tok_s"], 3),
                           "decode_ratio": round(a["decode_tok_s"] / b["decode_tok_s"], 3)}
    line = {"metric": f"{design} vs {beside} at equal layer sizes, tokens/s ratio ({layers} layers, eager steps)",
            "prefill_tokens": prefill, "decode_batch": batch, "decode_context": context, "ratios": summary}
    print(json.dumps(line), flush=True)
    return line
