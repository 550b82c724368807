"""Plain, slow implementation of the Livitar design, one function per mechanism, token by token where a
mechanism is recurrent. It shares no code with ``vgate``: tests compare the engine against it.

A model is (cfg, tensors): ``cfg`` the dict of config.json, ``tensors`` name -> torch tensor. Everything is
computed in ``DT`` (float64 by default) from the tensors' values.
"""
from __future__ import annotations

import math

import torch

DT = torch.float64


def _t(x):
    return x.to(DT)


def tanh_norm(x, tensors, name):
    """y = tanh(alpha x) * w + b: a norm without statistics."""
    return torch.tanh(_t(tensors[name + ".alpha"]) * x) * _t(tensors[name]) + _t(tensors[name + ".b"])


def unit_rms(x, eps):
    """x over sqrt(mean(x^2) + eps) along the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def turn_halves(x, pos, dims, base):
    """Rotary positions in the half-split layout: entry i < dims/2 is paired with entry i + dims/2.
    x [n, heads, d], pos [n]."""
    half = dims // 2
    y = x.clone()
    if half == 0:
        return y
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=DT)
    ang = pos.to(DT)[:, None, None] * f
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:dims]
    y[..., :half] = a * c - b * s
    y[..., half:dims] = b * c + a * s
    return y


def retention(h, m, tensors, pre, eps, pos0=0, state=None):
    """Decayed linear attention, one token after the other. Returns (output [n, width], state [H, D, V])."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = (h @ _t(tensors[pre + "q"]).T).view(n, H, D)
    k = (h @ _t(tensors[pre + "k"]).T).view(n, H, D)
    v = (h @ _t(tensors[pre + "v"]).T).view(n, H, V)
    pos = torch.arange(pos0, pos0 + n)
    rot = m["rot"]
    q = turn_halves(q, pos, rot["dims"], rot["base"])
    k = turn_halves(k, pos, rot["dims"], rot["base"]) * D ** -0.5
    S = torch.zeros(H, D, V, dtype=DT) if state is None else state.clone()
    dec = torch.tensor(m["decay"], dtype=DT)
    o = torch.empty(n, H, V, dtype=DT)
    for t in range(n):
        S = dec[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps).reshape(n, H * V)
    g = h @ _t(tensors[pre + "g"]).T
    o = o * (g * torch.sigmoid(g))
    return o @ _t(tensors[pre + "o"]).T, S


def rel_bucket(n: int, B: int, far: float) -> int:
    """Row of the learned distance table for distance n: one row per distance below B/2, then rows spaced
    evenly in log(distance) up to ``far``."""
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half))))


def attend(q, k, v, bias):
    """Causal softmax attention of one head; q [n, D] at positions pos0 .. pos0 + n - 1 over keys k [m, D] at
    positions 0 .. m - 1 (m = pos0 + n); bias [n, m] is added to the scores (already scaled)."""
    n, m = q.shape[0], k.shape[0]
    pos0 = m - n
    sc = q @ k.T + bias
    i = torch.arange(pos0, m)[:, None]
    j = torch.arange(m)[None, :]
    sc = sc.masked_fill(j > i, float("-inf"))
    return torch.softmax(sc, -1) @ v


def attention(h, m, tensors, pre, eps, kind, keys=None, values=None):
    """The two softmax mixers. ``kind`` "attention": per-head temperature and a logarithmic distance
    penalty; "attention_2": unit-RMS queries and keys, a query temperature that grows with the position,
    and a learned bias per distance bucket. keys / values: what earlier tokens left ([m0, G, D], [m0, G, V]).
    Returns (output, keys, values)."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = (h @ _t(tensors[pre + "q"]).T).view(n, H, D)
    k = (h @ _t(tensors[pre + "k"]).T).view(n, G, D)
    v = (h @ _t(tensors[pre + "v"]).T).view(n, G, V)
    pos0 = 0 if keys is None else keys.shape[0]
    pos = torch.arange(pos0, pos0 + n)
    if kind == "attention_2":
        q, k = unit_rms(q, eps), unit_rms(k, eps)
        qt = m["q_temp"]
        grow = 1.0 + qt["coef"] * torch.log(torch.floor((pos + 1).to(DT) / qt["every"]) + 1.0)
        q = q * grow[:, None, None]
    if keys is not None:
        k, v = torch.cat([keys, k]), torch.cat([values, v])
    mtot = k.shape[0]
    dist = (pos[:, None] - torch.arange(mtot)[None, :]).clamp(min=0)      # [n, m]; future keys are masked anyway
    out = torch.empty(n, H, V, dtype=DT)
    rep = H // G
    for hd in range(H):
        if kind == "attention":
            r1, r2, temp = (float(_t(tensors[pre + x])[hd]) for x in ("r1", "r2", "temp"))
            scale = m["scale"] * temp
            bias = -r1 * torch.log(1.0 + r2 * dist.to(DT))
        else:
            rel = _t(tensors[pre + "rel"])
            B = rel.shape[0]
            rows = torch.tensor([[rel_bucket(int(d), B, m["bias_max"]) for d in row] for row in dist.tolist()])
            scale = m["scale"]
            bias = rel[:, hd][rows]
        out[:, hd] = attend(q[:, hd] * scale, k[:, hd // rep], v[:, hd // rep], bias)
    o = out.reshape(n, H * V) * torch.sigmoid(h @ _t(tensors[pre + "g"]).T)
    return o @ _t(tensors[pre + "o"]).T, k, v


def gated_ff(h, tensors, pre):
    g = h @ _t(tensors[pre + "gate"]).T
    return ((g * torch.sigmoid(g)) * (h @ _t(tensors[pre + "up"]).T)) @ _t(tensors[pre + "down"]).T


def experts_ff(h, mlp, tensors, pre):
    """Softmax router over all experts, the ``top`` largest chosen, their scores renormalised and scaled;
    plus a shared expert every token runs."""
    r = mlp["router"]
    z = h @ _t(tensors[pre + "router"]).T
    s = torch.softmax(z, -1)
    top_s, top_i = torch.topk(s, r["top"], dim=-1)
    w = top_s / (top_s.sum(-1, keepdim=True) + 1e-20) * r["scale"]
    out = torch.zeros(h.shape[0], tensors[pre + "e0.down"].shape[0], dtype=DT)
    for t in range(h.shape[0]):
        for c in range(r["top"]):
            out[t] += w[t, c] * gated_ff(h[t:t + 1], tensors, f"{pre}e{int(top_i[t, c])}.")[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, tensors, pre + "shared.")
    return out


def hyper_step(xs, tensors, pre, sublayer, norm):
    """One sublayer over the stream copies xs [s, n, width]: read a weighted sum of the copies, run the
    sublayer on its norm, then mix the copies among themselves and add the result to each with its own weight."""
    u = torch.einsum("s,snw->nw", _t(tensors[pre + "in"]), xs)
    y = sublayer(norm(u))
    mix = _t(tensors[pre + "mix"])          # [from, to]
    return torch.einsum("st,snw->tnw", mix, xs) + _t(tensors[pre + "out"])[:, None, None] * y[None]


def forward(cfg, tensors, tokens, carry=None, per_layer=None):
    """Logits [n, vocab] of ``tokens`` (list of ints) continuing from ``carry`` (what :func:`forward`
    returned for the tokens before them; None at a sequence's start). Returns (logits, carry)."""
    eps = cfg["norm"]["eps"]
    n = len(tokens)
    x = _t(tensors["embed"])[torch.tensor(tokens)]
    xs = x[None].repeat(cfg["streams"], 1, 1)
    pos0 = 0 if carry is None else carry["n"]
    new = {"n": pos0 + n, "layers": []}
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        old = None if carry is None else carry["layers"][i]
        kept = {}

        def mixer(hn, L=L, pre=pre, old=old, kept=kept):
            if L["type"] == "retention":
                y, kept["S"] = retention(hn, L["mixer"], tensors, pre + "mix.", eps, pos0, None if old is None else old["S"])
            else:
                y, kept["k"], kept["v"] = attention(hn, L["mixer"], tensors, pre + "mix.", eps, L["type"],
                                                    None if old is None else old["k"], None if old is None else old["v"])
            return y

        xs = hyper_step(xs, tensors, pre + "hc1.", mixer, lambda u, pre=pre: tanh_norm(u, tensors, pre + "norm1"))
        if L.get("mlp"):
            xs = hyper_step(xs, tensors, pre + "hc2.", lambda hn, L=L, pre=pre: experts_ff(hn, L["mlp"], tensors, pre + "mlp."),
                            lambda u, pre=pre: tanh_norm(u, tensors, pre + "norm2"))
        new["layers"].append(kept)
        if per_layer is not None:
            per_layer.append(xs.sum(0))
    x = xs.sum(0)
    return tanh_norm(x, tensors, "final.norm") @ _t(tensors["head"]).T, new
