"""Plain, slow implementation of the Gefudra design, one function per mechanism, token by token where
recurrent. It shares no code with ``vgate`` and is what tests/test_gefudra.py holds the engine against.

Everything is float64 (``dt``) on the CPU; ``cfg`` is the parsed config.json, ``t`` a dict name -> tensor.
"""
from __future__ import annotations

import math

import torch

dt = torch.float64


def rms(x: torch.Tensor, eps: float, w: torch.Tensor | None = None) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w.to(dt)


def lin(w: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    return x @ w.to(dt).t()


def sink_softmax(s: torch.Tensor, sink: float | None) -> torch.Tensor:
    """Weights over the last axis of ``s``; with a sink the denominator has exp(sink) once more."""
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.clamp(m, min=float(sink))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(torch.tensor(float(sink), dtype=dt) - m)
    return e / den


def turn_halves(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [n, ..., d]: entry i of the first ``dims`` entries is paired with entry i + dims / 2 and the pair is
    turned by pos * base^(-2 i / dims)."""
    y = x.clone()
    half = dims // 2
    for i in range(half):
        a = pos.to(dt) * float(base) ** (-2.0 * i / dims)
        c, s = torch.cos(a), torch.sin(a)
        shape = [x.shape[0]] + [1] * (x.dim() - 2)
        c, s = c.view(shape), s.view(shape)
        u, v = x[..., i], x[..., i + half]
        y[..., i] = u * c - v * s
        y[..., i + half] = v * c + u * s
    return y


def latent_attention(m: dict, t: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """h [n, W] -> [n, W]; keys and values are made from one shared low-rank row per token."""
    n = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    win = m["mask"]["size"]
    q = lin(t["uq"], rms(lin(t["dq"], h), eps, t["dq.norm"])).view(n, H, D)
    c = rms(lin(t["dkv"], h), eps, t["dkv.norm"])
    k = lin(t["uk"], c).view(n, H, D)
    v = lin(t["uv"], c).view(n, H, V)
    out = torch.zeros(n, H, V, dtype=dt)
    for i in range(n):
        lo = max(0, i - win + 1)
        for hd in range(H):
            s = (k[lo:i + 1, hd] @ q[i, hd]) * m["scale"]
            p = sink_softmax(s, float(t["sink"][hd]))
            out[i, hd] = p @ v[lo:i + 1, hd]
    out = out.reshape(n, H * V) * torch.sigmoid(lin(t["g"], h))
    return lin(t["o"], out)


def diff_attention(m: dict, t: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """Two softmax maps per head over the same values, the second subtracted with one learned factor."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = turn_halves(lin(t["q"], h).view(n, H, 2, D), pos, rot["dims"], rot["base"])
    k = turn_halves(lin(t["k"], h).view(n, G, 2, D), pos, rot["dims"], rot["base"])
    v = lin(t["v"], h).view(n, G, V)
    lam = (math.exp(float((t["lq1"].to(dt) * t["lk1"].to(dt)).sum()))
           - math.exp(float((t["lq2"].to(dt) * t["lk2"].to(dt)).sum())) + m["diff"])
    cap = m["softcap"]
    out = torch.zeros(n, H, V, dtype=dt)
    for i in range(n):
        for hd in range(H):
            g = hd // (H // G)
            a = []
            for mp in range(2):
                s = (k[:i + 1, g, mp] @ q[i, hd, mp]) * m["scale"]
                s = cap * torch.tanh(s / cap)
                a.append(sink_softmax(s, None) @ v[:i + 1, g])
            o = a[0] - lam * a[1]
            out[i, hd] = rms(o, eps) * (1.0 - m["diff"])
    out = out.reshape(n, H * V) * torch.sigmoid(lin(t["g"], h))
    return lin(t["o"], out)


def wkv(m: dict, t: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """Decayed outer-product state per head with a bonus for the current token; inputs are blends of the
    token's and the previous token's row."""
    n, W = h.shape
    H, D = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, W, dtype=dt), h[:-1]])
    mix = {s: h + (prev - h) * t["mu." + s].to(dt) for s in "rkvgw"}
    r = lin(t["r"], mix["r"]).view(n, H, D)
    k = lin(t["k"], mix["k"]).view(n, H, D)
    v = lin(t["v"], mix["v"]).view(n, H, D)
    gate = torch.nn.functional.silu(lin(t["g"], mix["g"]))
    w = torch.exp(-torch.exp(lin(t["w2"], torch.tanh(lin(t["w1"], mix["w"]))) + t["w0"].to(dt))).view(n, H, D)
    u = t["u"].to(dt).view(H, D)
    S = torch.zeros(H, D, D, dtype=dt)
    out = torch.zeros(n, H, D, dtype=dt)
    for i in range(n):
        kv = k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[i])
        S = w[i][:, :, None] * S + kv
    out = rms(out, eps).reshape(n, H * D) * t["norm"].to(dt) * gate
    return lin(t["o"], out)


def feed_forward(m: dict, t: dict, h: torch.Tensor) -> torch.Tensor:
    L = m["limit"]
    g = torch.clamp(lin(t["gate"], h), max=L)
    u = torch.clamp(lin(t["up"], h), -L, L)
    return lin(t["down"], g * torch.sigmoid(1.702 * g) * (u + 1.0))


MIXERS = {"latent_attention": latent_attention, "attention": diff_attention, "wkv": wkv}


def sub(t: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in t.items() if k.startswith(prefix)}


def run_order(cfg: dict) -> list:
    """(layer index, first of a pass) in the order the layers run."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, times = lp["start"], lp["stop"], lp["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg: dict, t: dict, tokens: list) -> tuple:
    """(logits [n, vocab], residual stream after every layer run [runs, n, W])."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x0 = t["embed"].to(dt)[torch.tensor(tokens)]
    x = x0.clone()
    streams = []
    for i, first in run_order(cfg):
        L = cfg["layers"][i]
        lt = sub(t, f"l{i}.")
        if first:
            x = lin(t["loop.in"], torch.cat([x, x0], -1))
        x = x + mult * MIXERS[L["type"]](L["mixer"], sub(lt, "mix."), eps, rms(x, eps, lt["norm1"]))
        if L.get("mlp"):
            x = x + mult * feed_forward(L["mlp"], sub(lt, "mlp."), rms(x, eps, lt["norm2"]))
        streams.append(x.clone())
    logits = lin(t["embed"], rms(x, eps, t["final.norm"])) * cfg["logit_scale"]
    return logits, torch.stack(streams)
