"""Ops of layered hybrid models (fp32 residual stream, bf16 or fp32 activations).

Same dispatch rule as the rest of :mod:`vgate.ops`: GPU tensors go to the HIP kernels
(csrc/kernels/gemm_any.hip, seq_elementwise.hip, latent_attn.hip, delta_rule.hip) and raise if the
extension is missing; CPU tensors run the unfused torch forms below (the CPU device of tests).
Everything the kernels compute in fp32 is fp32 here too; rows are rounded to the activation dtype
at the same places.
"""
from __future__ import annotations

import math
import os

import torch


class _Traced:
    """VGATE_SEQ_TRACE=1: print every kernel call (name, shapes) before it is launched and wait for
    it, so a failing launch is named by the last line printed."""

    def __init__(self, mod):
        self._mod = mod

    def __getattr__(self, name):
        fn = getattr(self._mod, name)

        def call(*a, **k):
            shapes = [tuple(x.shape) if isinstance(x, torch.Tensor) else x for x in a]
            print(f"[seq] {name} {shapes}", flush=True)
            out = fn(*a, **k)
            torch.cuda.synchronize()
            return out
        return call


_TRACE = os.environ.get("VGATE_SEQ_TRACE", "0") == "1"


def _C():
    from vgate import ops
    mod = ops.native()
    return _Traced(mod) if _TRACE else mod


ACT_NONE, ACT_SILU_MUL, ACT_CLAMPED_GLU, ACT_TANH, ACT_GELU_TANH_MUL = 0, 1, 2, 3, 4
BIAS_NONE, BIAS_LOG, BIAS_TABLE = 0, 1, 2   # distance term of an attention score (see window_attn)
MAX_STREAMS = 16            # copies of the residual stream hyper_mix takes
WINDOW_SPLIT = os.environ.get("VGATE_WINDOW_SPLIT", "1") == "1"   # "0": one workgroup per decoded 16-row tile
LATENT_SPLIT = os.environ.get("VGATE_LATENT_SPLIT", "1") == "1"   # "0": one workgroup per decoded sequence
LINEAR_ATTN_MAX_DIM = 256   # key channels per head the recurrence kernel keeps in registers (csrc/kernels/linear_attn.hip)


def _act(g: torch.Tensor, u: torch.Tensor | None, act: int, limit: float, alpha: float) -> torch.Tensor:
    if act == ACT_SILU_MUL:
        return g * torch.sigmoid(g) * u
    if act == ACT_CLAMPED_GLU:
        g = g.clamp(max=limit)
        u = u.clamp(-limit, limit)
        return g * torch.sigmoid(alpha * g) * (u + 1.0)
    if act == ACT_TANH:
        return torch.tanh(g)
    if act == ACT_GELU_TANH_MUL:
        return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g))) * u
    return g


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, w2: torch.Tensor | None = None,
         bias: torch.Tensor | None = None, gate: torch.Tensor | None = None, a_rows: torch.Tensor | None = None,
         group_off: torch.Tensor | None = None, act: int = 0, limit: float = 0.0, alpha: float = 1.702) -> torch.Tensor:
    """out = epi(a @ w^T): 2-D, batched (3-D a / w / out) or grouped (2-D a / out, 3-D w, device row
    ranges ``group_off``; rows of a gathered through ``a_rows``). Epilogue: + bias, activation (pair
    forms take ``w2``), * sigmoid(gate). fp32 accumulation; one rounding to out's dtype."""
    if a.is_cuda:
        _C().gemm_any(a, w, out, w2, bias, gate, a_rows, group_off, act, limit, alpha)
        return out
    af, wf = a.float(), w.float()
    if group_off is not None:
        off = group_off.tolist()
        res = torch.zeros(out.shape, dtype=torch.float32)
        for g in range(w.shape[0]):
            lo, hi = off[g], off[g + 1]
            if hi <= lo:
                continue
            rows = af[a_rows[lo:hi].long()] if a_rows is not None else af[lo:hi]
            y = rows @ wf[g].t()
            u = rows @ w2[g].float().t() if w2 is not None else None
            res[lo:hi] = _act(y, u, act, limit, alpha)
        out.copy_(res)
        return out
    M = out.shape[-2]
    af = af[a_rows[:M].long()] if a_rows is not None else af[..., :M, :]
    y = af @ wf.transpose(-1, -2)
    if bias is not None:
        y = y + bias
    u = af @ w2.float().transpose(-1, -2) if w2 is not None else None
    y = _act(y, u, act, limit, alpha)
    if gate is not None:
        y = y * torch.sigmoid(gate[..., :M, :].float())
    out.copy_(y)
    return out


def norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor, rows: torch.Tensor | None = None,
              scalar: bool = False) -> torch.Tensor:
    """out[m] = x[rows[m]] / sqrt(mean(x^2) + eps) * w (w fp32: one number if ``scalar``)."""
    if x.is_cuda:
        _C().norm_rows(x, w, eps, out, rows, scalar)
        return out
    xf = x.float()
    xf = xf[rows.long()] if rows is not None else xf[: out.shape[0]]
    y = xf * (1.0 / torch.sqrt(xf.pow(2).mean(-1, keepdim=True) + eps)) * w
    out.copy_(y)
    return out


def embed_rows(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, prev: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 rows of the embedding table; ids < 0 name the previous step's sample prev[-id - 1]."""
    if table.is_cuda:
        _C().embed_rows(ids, table, out, prev)
        return out
    if prev is not None and bool((ids < 0).any()):
        ids = torch.where(ids < 0, prev.to(ids.device)[(-ids - 1).clamp(min=0).long()], ids)
    out.copy_(table[ids.long()].float())
    return out


def gated_residual(x, y1, g1=None, b1=None, y2=None, g2=None, b2=None) -> None:
    """x += y1 * sigmoid(g1 + b1) [+ y2 * sigmoid(g2 + b2)] in fp32 (g: strided column views)."""
    if x.is_cuda:
        _C().gated_residual(x, y1, g1, b1, y2, g2, b2)
        return
    T = x.shape[0]
    v = y1.float()
    if g1 is not None:
        v = v * torch.sigmoid(g1[:T].float() + (b1 if b1 is not None else 0.0))
    if y2 is not None:
        u = y2.float()
        if g2 is not None:
            u = u * torch.sigmoid(g2[:T].float() + (b2 if b2 is not None else 0.0))
        v = v + u
    x += v


def rope_inv_freq(dims: int, base: float, device, scaling: dict | None = None) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2, rounded to fp32 once. ``scaling`` {factor, low, high,
    original} stretches long wavelengths (the Llama-3.1 rule): with l = 2 pi / f, f is kept where
    l < original / high, divided by factor where l > original / low, and blended linearly in
    original / l between the two."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wl = 2.0 * math.pi / f
            if wl > orig / low:
                f = f / factor
            elif wl >= orig / high:
                s = (orig / wl - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float32).to(device)


def _rope_pairs(x: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor, dims: int) -> torch.Tensor:
    """Rotate the leading ``dims`` entries of the last axis in interleaved pairs (2i, 2i + 1); fp32."""
    y = x.clone()
    if dims == 0:
        return y
    ang = pos.float()[:, None] * inv_freq[None]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    return y


def _rope_halves(x: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor, dims: int) -> torch.Tensor:
    """Rotate the leading ``dims`` entries of the last axis, entry i paired with entry i + dims / 2; fp32."""
    y = x.clone()
    if dims == 0:
        return y
    half = dims // 2
    ang = pos.float()[:, None] * inv_freq[None, :half]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    y[..., :half] = u * c - v * s
    y[..., half:dims] = v * c + u * s
    return y


def latent_write(kv, w, eps, positions, slots, inv_freq, rot_dims: int, cache, rank: int, cache_t=None) -> None:
    """cache[slot] = [rmsnorm(kv[:rank]) * w, rope(kv[rank:])] for every token with slot >= 0.
    ``cache_t`` (GPU, bf16): a second copy of the latent part laid out [page, column, key in page], the
    operand layout of the MFMA attention kernel's weighted sum."""
    if kv.is_cuda:
        _C().latent_write(kv, w, eps, positions, slots, inv_freq, rot_dims, cache, rank, cache_t)
        return
    x = kv.float()
    c = x[:, :rank]
    c = c * (1.0 / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps)) * w
    kr = _rope_pairs(x[:, rank:], positions, inv_freq, rot_dims)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok].long()] = row[ok]


def latent_qrope(q, positions, inv_freq, rot_dims: int, qa, H: int, dim: int, rank: int, rot: int) -> None:
    """qa[t, h, rank:] = rope(q[t, h, dim:])."""
    if q.is_cuda:
        _C().latent_qrope(q, positions, inv_freq, rot_dims, qa, H, dim, rank, rot)
        return
    T = q.shape[0]
    qr = q.view(T, H, dim + rot)[..., dim:].float()
    qa.view(T, H, rank + rot)[..., rank:] = _rope_pairs(qr, positions, inv_freq, rot_dims).to(qa.dtype)


LATENT_FULL = 1 << 30   # "window" of a latent attention that sees every earlier position


def latent_attn(qa, cache, block_tables, context_lens, query_start, ol, scale: float, H: int, rank: int, rot: int,
                num_seqs: int | None = None, cache_t=None, window: int = LATENT_FULL, sink=None) -> None:
    """ol[t, h] = sum_j softmax_j(scale * qa[t, h] . cache_j) cache_j[:rank] over the keys j with
    0 <= position(t) - j < window. ``sink`` [H] fp32: exp(sink[h]) is added to the softmax denominator (unscaled,
    once). With ``cache_t`` (see :func:`latent_write`) bf16 caches run the MFMA kernel."""
    if qa.is_cuda:
        parts, scratch = 1, None
        if cache_t is not None and LATENT_SPLIT:   # decoded tokens of the MFMA kernel: several workgroups per sequence
            T = qa.numel() // (H * (rank + rot))
            parts, n = _C().latent_attn_split(T, block_tables.shape[0], H, rank, rot, cache.dtype == torch.float32, cache.shape[1])
            if parts > 1:
                scratch = torch.empty(n, dtype=torch.float32, device=qa.device)
        _C().latent_attn(qa, cache, block_tables, context_lens, query_start, ol, scale, H, rank, rot, cache_t, window, sink,
                         parts, scratch)
        return
    E = rank + rot
    T = qa.numel() // (H * E)
    q3 = qa.view(T, H, E).float()
    o3 = ol.view(T, H, rank)
    page = cache.shape[1]
    S = block_tables.shape[0] if num_seqs is None else num_seqs
    flat = cache.view(-1, E)
    for s in range(S):
        t0, t1 = int(query_start[s]), int(query_start[s + 1])
        if t1 <= t0:
            continue
        ctx = int(context_lens[s])
        j = torch.arange(ctx)
        rows = flat[(block_tables[s].long()[j // page] * page + j % page)].float()
        sc = torch.einsum("the,je->thj", q3[t0:t1], rows) * scale
        pos = ctx - (t1 - t0) + torch.arange(t1 - t0)
        hidden = (j[None, None, :] > pos[:, None, None]) | (j[None, None, :] <= pos[:, None, None] - window)
        sc = sc.masked_fill(hidden, float("-inf"))
        if sink is not None:
            sc = torch.cat([sc, sink.view(1, H, 1).expand(t1 - t0, H, 1)], -1)
        p = torch.softmax(sc, -1)[..., :ctx]
        o3[t0:t1] = torch.einsum("thj,jr->thr", p, rows[:, :rank]).to(ol.dtype)


def delta_rule(r, k, v, g, a, wl, w0, ab, nw, state, state_slots, context_lens, query_start, out,
               decay_c: float, unit_eps: float, eps: float, num_seqs: int | None = None) -> None:
    """Generalized delta rule over state slots (see csrc/kernels/delta_rule.hip); state [slots, H, D, D]."""
    if r.is_cuda:
        scratch = torch.empty(6 * r.shape[0] * r.shape[1], dtype=torch.float32, device=r.device)
        _C().delta_rule(r, k, v, g, a, wl, w0, ab, nw, state, state_slots, context_lens, query_start, out,
                        decay_c, unit_eps, eps, scratch)
        return
    H, D = state.shape[1], state.shape[2]
    S = state_slots.numel() if num_seqs is None else num_seqs
    for s in range(S):
        t0, t1 = int(query_start[s]), int(query_start[s + 1])
        slot = int(state_slots[s])
        if t1 <= t0 or slot < 0:
            continue
        pos0 = int(context_lens[s]) - (t1 - t0)
        St = state[slot].clone() if pos0 > 0 else torch.zeros(H, D, D)

        def hd(x):
            return x[t0:t1].float().view(t1 - t0, H, D)

        rr, kk, vv, gg = hd(r), hd(k), hd(v), hd(g)
        w = torch.exp(-decay_c * torch.sigmoid(hd(wl) + w0.view(H, D)))
        al = torch.sigmoid(hd(a) + ab.view(H, D))
        u = kk * (1.0 / torch.sqrt(kk.pow(2).sum(-1, keepdim=True) + unit_eps))
        for i in range(t1 - t0):
            uS = torch.einsum("hk,hkv->hv", u[i], St)
            St = w[i][:, :, None] * St - (al[i] * u[i])[:, :, None] * uS[:, None, :] + kk[i][:, :, None] * vv[i][:, None, :]
            o = torch.einsum("hkv,hk->hv", St, rr[i])
            o = o * (1.0 / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps)) * nw.view(H, D) * torch.sigmoid(gg[i])
            out[t0 + i] = o.reshape(H * D).to(out.dtype)
        state[slot] = St


def moe_route(z, corr, top: int, norm_eps: float, idx, wts, softmax: bool = False, scale: float = 1.0) -> None:
    """idx / wts [T, top]: the ``top`` largest of s + corr with s = sigmoid(z), or softmax(z) over all
    experts; weights s of the chosen over (their sum + norm_eps), times ``scale``."""
    if z.is_cuda:
        _C().moe_route(z, corr, top, norm_eps, idx, wts, softmax, scale)
        return
    s = torch.softmax(z, -1) if softmax else torch.sigmoid(z)
    choice = s + corr if corr is not None else s
    # arg-max rounds, lowest index first on ties (the kernel's order)
    c = choice.clone()
    picks = []
    for _ in range(top):
        i = c.argmax(-1)
        picks.append(i)
        c.scatter_(1, i[:, None], float("-inf"))
    ii = torch.stack(picks, 1)
    ws = torch.gather(s, 1, ii)
    idx.copy_(ii.int())
    wts.copy_(ws / (ws.sum(-1, keepdim=True) + norm_eps) * scale)


def moe_sort(idx, E: int, rows, pos, off) -> None:
    """Group the (token, choice) pairs by expert: rows[p] = token, pos[t, c] = p, off[E + 1]."""
    if idx.is_cuda:
        _C().moe_sort(idx, E, rows, pos, off)
        return
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    top = idx.shape[1]
    rows.copy_((order // top).int())
    p = torch.empty_like(order)
    p[order] = torch.arange(order.numel())
    pos.copy_(p.int().view(pos.shape))
    cnt = torch.bincount(flat, minlength=E)
    off.copy_(torch.cat([torch.zeros(1, dtype=torch.long), cnt.cumsum(0)]).int())


def moe_combine(y, pos, wts, out, add=None) -> None:
    """out[t] = sum_c wts[t, c] * y[pos[t, c]] [+ add[t]] (fp32 sum; out bf16 or fp32)."""
    if y.is_cuda:
        _C().moe_combine(y, pos, wts, out, add)
        return
    T, top = wts.shape
    rows = y.float()[pos.view(T, top).long()]
    r = (rows * wts[:, :, None]).sum(1)
    out.copy_(r if add is None else r + add[:T].float())


# ------------------------------------------------------------------ post-norm residual, depth average
def cast_rows(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = x rounded to out's dtype (the copy of the fp32 stream a bf16 GEMM reads)."""
    if x.is_cuda:
        _C().cast_rows(x, out)
        return out
    out.copy_(x[: out.shape[0]])
    return out


def tanh_norm_rows(x: torch.Tensor, alpha: torch.Tensor, w: torch.Tensor, b: torch.Tensor, out: torch.Tensor,
                   rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[m] = tanh(alpha * x[rows[m]]) * w + b: a norm without statistics (alpha one fp32 number, w / b
    fp32 vectors), computed in fp32 and rounded to out's dtype."""
    if x.is_cuda:
        _C().tanh_norm_rows(x, alpha, w, b, out, rows)
        return out
    xf = x.float()
    xf = xf[rows.long()] if rows is not None else xf[: out.shape[0]]
    out.copy_(torch.tanh(alpha * xf) * w + b)
    return out


def hyper_mix(xs: torch.Tensor, y: torch.Tensor | None, mix: torch.Tensor | None, out_w: torch.Tensor | None,
              read_w: torch.Tensor | None = None, alpha=None, w=None, b=None, h_out: torch.Tensor | None = None,
              sum_out: torch.Tensor | None = None) -> None:
    """One sublayer's write to ``xs`` [S, T, W] (fp32 copies of the residual stream), fused with the next
    sublayer's read. With ``y`` [T, W]: all copies at once from the old ones,
        xs[t] <- sum_s mix[s, t] xs[s] + out_w[t] * y.
    With ``read_w`` [S]: u = sum_s read_w[s] xs[s] (the new copies), h_out = tanh(alpha u) * w + b in h_out's
    dtype. With ``sum_out`` [T, W] fp32: the sum of the (new) copies. Everything in fp32."""
    if xs.is_cuda:
        _C().hyper_mix(xs, y, mix, out_w, read_w, alpha, w, b, h_out, sum_out)
        return
    if y is not None:
        T = y.shape[0]
        new = torch.einsum("st,snw->tnw", mix, xs[:, :T]) + out_w[:, None, None] * y.float()[None]
        xs[:, :T] = new
    if read_w is not None:
        T = h_out.shape[0]
        u = torch.einsum("s,snw->nw", read_w, xs[:, :T])
        h_out.copy_(torch.tanh(alpha * u) * w + b)
    if sum_out is not None:
        sum_out.copy_(xs[:, : sum_out.shape[0]].sum(0))


def glu_rows(gu: torch.Tensor, out: torch.Tensor, act: int, limit: float = 0.0, alpha: float = 1.702) -> torch.Tensor:
    """out = act(gu[:, :n], gu[:, n:]) for a stacked [gate; up] projection (act: ACT_SILU_MUL, ACT_GELU_TANH_MUL, or
    ACT_CLAMPED_GLU with ``limit`` and ``alpha``)."""
    if gu.is_cuda:
        _C().glu_rows(gu, out, act, limit, alpha)
        return out
    n = out.shape[1]
    out.copy_(_act(gu[: out.shape[0], :n].float(), gu[: out.shape[0], n:].float(), act, limit, alpha))
    return out


def residual_norm(x: torch.Tensor, y: torch.Tensor, mult: float, w: torch.Tensor | None = None, eps: float = 0.0,
                  h_out: torch.Tensor | None = None) -> None:
    """x += mult * y in fp32 (x fp32 [T, W], y fp32 or the activation dtype). With ``w`` [W]: also
    h_out = x / sqrt(mean(x^2) + eps) * w from the new x, rounded to h_out's dtype."""
    if x.is_cuda:
        _C().residual_norm(x, y, mult, w, eps, h_out)
        return
    T = y.shape[0]
    x[:T] += mult * y.float()
    if w is not None:
        xf = x[: h_out.shape[0]]
        h_out.copy_(xf * (1.0 / torch.sqrt(xf.pow(2).mean(-1, keepdim=True) + eps)) * w)


def pair_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = [a[t], b[t]] (two fp32 [T, W] row sets side by side) rounded to out's dtype."""
    if a.is_cuda:
        _C().pair_rows(a, b, out)
        return out
    T = out.shape[0]
    out.copy_(torch.cat([a[:T], b[:T]], -1))
    return out


def shift_mix(h: torch.Tensor, last: torch.Tensor, mu: torch.Tensor, state_slots, context_lens, query_start,
              out: torch.Tensor, num_seqs: int | None = None) -> None:
    """Blends of every token's row with the row of the token before it: out[s, t] = h[t] + (h'[t] - h[t]) * mu[s]
    for the ``mu`` [n, W] fp32 blend vectors, with h' the previous token's h: the row before inside the step, the
    sequence's ``last`` [slots, W] fp32 row for the first token of a portion, zeros at position 0. Afterwards
    ``last`` holds the portion's last row. Computed in fp32, rounded once to out's dtype."""
    if h.is_cuda:
        _C().shift_mix(h, last, mu, state_slots, context_lens, query_start, out)
        return
    S = state_slots.numel() if num_seqs is None else num_seqs
    for s in range(S):
        t0, t1 = int(query_start[s]), int(query_start[s + 1])
        slot = int(state_slots[s])
        if t1 <= t0 or slot < 0:
            continue
        hf = h[t0:t1].float()
        first = last[slot].clone() if int(context_lens[s]) - (t1 - t0) > 0 else torch.zeros_like(last[slot])
        prev = torch.cat([first[None], hf[:-1]])
        out[:, t0:t1] = (hf[None] + (prev - hf)[None] * mu[:, None, :]).to(out.dtype)
        last[slot] = hf[-1]


def map_pair_combine(a: torch.Tensor, lam: float, out_scale: float, eps: float, gate, out: torch.Tensor, H: int, G: int,
                     V: int) -> None:
    """Two attention maps per head into one output. ``a`` [T, 2 H V] holds the maps' results grouped (key/value
    head, map, head in group); per head h: o = a1 - lam * a2, o / sqrt(mean(o^2) + eps) over V, times
    ``out_scale``, times sigmoid(gate[t, h]) if given; out [T, H V] with the heads in their own order. fp32."""
    if a.is_cuda:
        _C().map_pair_combine(a, lam, out_scale, eps, gate, out, H, G, V)
        return
    T = out.shape[0]
    rep = H // G
    af = a[:T].float().view(T, G, 2, rep, V)
    o = (af[:, :, 0] - lam * af[:, :, 1]).reshape(T, H, V)
    o = o * (1.0 / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps)) * out_scale
    o = o.reshape(T, H * V)
    if gate is not None:
        o = o * torch.sigmoid(gate[:T].float())
    out.copy_(o)


def post_norm_add(x, y1, w, eps: float, out, s1: float = 1.0, y2=None, s2: float = 1.0, act_out=None, hist=None,
                  planes: int = 0, coef=None, mix=None) -> None:
    """out = x + u / sqrt(mean(u^2) + eps) * w with u = s1 y1 [+ s2 y2], all in fp32 (out may be x).
    With ``hist`` [n, T, W] (whose plane ``planes - 1`` is ``out``): mix = sum_{j < planes} coef[j] hist[j],
    the depth average. ``act_out``: a copy of mix (or of out without hist) in the activation dtype."""
    if x.is_cuda:
        _C().post_norm_add(x, y1, w, eps, out, s1, y2, s2, act_out, hist, planes, coef, mix)
        return
    T = out.shape[0]
    u = y1[:T].float() * s1
    if y2 is not None:
        u = u + y2[:T].float() * s2
    r = x[:T] + u * (1.0 / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps)) * w
    out.copy_(r)
    last = out
    if hist is not None:
        acc = torch.zeros_like(r)
        for j in range(planes):
            acc = acc + coef[j] * hist[j][:T]
        mix.copy_(acc)
        last = mix
    if act_out is not None:
        act_out.copy_(last)


# ---------------------------------------------------------------------------------- window attention
def _rope_pairs_heads(x: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor, dims: int, sign: float = 1.0):
    """x [T, heads, d]: the leading ``dims`` entries of every head turned in interleaved pairs by sign * pos * f_i."""
    return _rope_pairs(x, pos.float() * sign, inv_freq, dims)


def window_write(q, k, v, qw, kw, eps: float, norm_all: bool, positions, slots, inv_freq, rot_dims: int, v_freq,
                 kc, vc, q_out, H: int, G: int, vt=None, q_head_scale=None, q_temp_coef: float = 0.0,
                 q_temp_every: int = 1, rot_half: bool = False) -> None:
    """Prepare one step's queries, keys and values of a window-attention layer.
    q [T, H * D], k [T, G * D], v [T, G * V] (biases already added). Query / key RMS norm (``qw`` / ``kw``
    None: none; ``norm_all``: over the whole projection with a [heads * D] weight, else per head with a
    [D] weight), rotation of the first ``rot_dims`` entries of every head, values turned over all of V
    by ``v_freq`` if given. Query temperatures (fp32, after the norm): head h times ``q_head_scale`` [h], the
    query at position p times 1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1). q goes to ``q_out``; keys and values to the paged caches
    kc [pages, G, page, D] / vc [pages, G, page, V] at the tokens' slots (slot < 0: padding row).
    ``vt`` (GPU, bf16): a second copy of the values laid out [pages, G, V, page], the operand layout of
    the MFMA attention kernel's weighted sum. ``rot_half``: entry i is paired with entry i + rot_dims / 2 instead
    of 2i with 2i + 1. The value cache may have fewer heads than the key cache (vc.shape[1] divides G: consecutive
    key heads share a value head); v then is [T, value heads * V]."""
    if q.is_cuda:
        _C().window_write(q, k, v, qw, kw, eps, norm_all, positions, slots, inv_freq, rot_dims, v_freq, kc, vc, q_out, H, G, vt,
                          q_head_scale, q_temp_coef, q_temp_every, rot_half)
        return
    T = q.shape[0]
    D, V, page = kc.shape[3], vc.shape[3], kc.shape[2]
    qf, kf, vf = q.float(), k.float(), v.float()

    def norm(x, w, heads):
        if w is None:
            return x.view(T, heads, D)
        if norm_all:
            return (x * (1.0 / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)) * w).view(T, heads, D)
        x = x.view(T, heads, D)
        return x * (1.0 / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)) * w

    turn = (lambda x: _rope_halves(x, positions[:T], inv_freq, rot_dims)) if rot_half else \
        (lambda x: _rope_pairs_heads(x, positions[:T], inv_freq, rot_dims))
    qn = turn(norm(qf, qw, H))
    if q_head_scale is not None:
        qn = qn * q_head_scale.view(1, H, 1)
    if q_temp_coef != 0.0:
        grow = 1.0 + q_temp_coef * torch.log(torch.floor((positions[:T] + 1).float() / q_temp_every) + 1.0)
        qn = qn * grow.view(T, 1, 1)
    kn = turn(norm(kf, kw, G))
    vn = vf.view(T, vc.shape[1], V)
    if v_freq is not None:
        vn = _rope_pairs_heads(vn, positions[:T], v_freq, 2 * v_freq.numel())
    q_out.copy_(qn.reshape(T, H * D))
    ok = slots[:T] >= 0
    sl = slots[:T][ok].long()
    kc[sl // page, :, sl % page] = kn[ok].to(kc.dtype)
    vc[sl // page, :, sl % page] = vn[ok].to(vc.dtype)


def _seq_rows(block_table: torch.Tensor, j: torch.Tensor, page: int):
    return block_table.long()[j // page], j % page


def window_pool(kc, vc, kp, vp, positions, block_tables, query_start, pool: int, num_seqs: int | None = None) -> None:
    """For every token of the step whose position completes a block of ``pool`` tokens: the mean of the
    block's cached keys (values) goes to kp (vp) [pages, G, ceil(page / pool), D], into the page of the
    block's last position e, row (e mod page) / pool."""
    if kc.is_cuda:
        _C().window_pool(kc, vc, kp, vp, positions, block_tables, query_start, pool)
        return
    page = kc.shape[2]
    S = block_tables.shape[0] if num_seqs is None else num_seqs
    for s in range(S):
        for t in range(int(query_start[s]), int(query_start[s + 1])):
            e = int(positions[t])
            if (e + 1) % pool:
                continue
            pg, r = _seq_rows(block_tables[s], torch.arange(e + 1 - pool, e + 1), page)
            dst = int(block_tables[s][e // page])
            kp[dst, :, (e % page) // pool] = kc[pg, :, r].float().mean(0).to(kp.dtype)
            vp[dst, :, (e % page) // pool] = vc[pg, :, r].float().mean(0).to(vp.dtype)


def window_attn(q, kc, vc, kp, vp, block_tables, context_lens, query_start, out, scale: float, H: int, window: int,
                pool: int, sink, v_freq, num_seqs: int | None = None, vt=None, prefill_kernel: int = 0,
                bias_kind: int = BIAS_NONE, bias_a=None, bias_b=None, gate=None, softcap: float = 0.0) -> None:
    """out[t, h] = sum_j p_j value_j over the keys position i of token t sees: the tokens j with
    0 <= i - j < window and, with ``pool`` = P > 0, the pooled row of every block b with
    b P + P - 1 <= i - window; p = softmax(scale q . key) over both kinds together, with exp(sink[h]) added
    to the denominator if ``sink`` is given. With ``v_freq`` the result is turned back by -i over all of V.
    Query head h reads key/value head h / (H / G). A distance term (no pooled blocks then) is added to the
    scaled score of the token at distance n = i - j: ``BIAS_LOG``: -bias_a[h] * ln(1 + bias_b[h] * n);
    ``BIAS_TABLE``: bias_a[h, min(n, last)] (fp32 [H, distances]). ``gate`` [T, H * V]: the result is
    multiplied by sigmoid(gate). With ``vt`` (see :func:`window_write`) bf16 caches run
    the MFMA kernels (``prefill_kernel``: which one prompt portions take, 0 = tiles staged in LDS for 64 rows,
    1 = 16 rows per workgroup with the tiles shared out over its waves). ``softcap`` c > 0: the scaled score s
    becomes c tanh(s / c) (not together with a distance term). The value caches may have fewer heads than the key
    cache (consecutive key heads share a value head)."""
    if q.is_cuda:
        parts, scratch = 1, None
        if vt is not None and WINDOW_SPLIT:   # decoded tokens of the MFMA kernel: several workgroups per 16-row tile
            parts, n = _C().window_attn_split(q.shape[0], block_tables.shape[0], H, kc.shape[1], kc.shape[3], vc.shape[3],
                                              kc.dtype == torch.float32, kc.shape[2])
            if parts > 1:
                scratch = torch.empty(n, dtype=torch.float32, device=q.device)
        _C().window_attn(q, kc, vc, kp, vp, block_tables, context_lens, query_start, out, scale, H, window, pool, sink, v_freq, vt,
                         prefill_kernel, bias_kind, bias_a, bias_b, gate, parts, scratch, softcap)
        return
    G, page, D, V = kc.shape[1], kc.shape[2], kc.shape[3], vc.shape[3]
    rep = H // G
    S = block_tables.shape[0] if num_seqs is None else num_seqs
    for s in range(S):
        t0, t1 = int(query_start[s]), int(query_start[s + 1])
        if t1 <= t0:
            continue
        pos0 = int(context_lens[s]) - (t1 - t0)
        bt = block_tables[s]
        for t in range(t0, t1):
            i = pos0 + t - t0
            lo = max(0, i - window + 1)
            pg, r = _seq_rows(bt, torch.arange(lo, i + 1), page)
            K, Vv = kc[pg, :, r].float(), vc[pg, :, r].float()           # [n, G, D], [n, value heads, V]
            if Vv.shape[1] != G:
                Vv = Vv.repeat_interleave(G // Vv.shape[1], dim=1)
            nb = max(0, i - window + 1) // pool if pool else 0
            if nb:
                e = torch.arange(nb) * pool + pool - 1
                pg, r = _seq_rows(bt, e, page)
                K = torch.cat([kp[pg, :, r // pool].float(), K])
                Vv = torch.cat([vp[pg, :, r // pool].float(), Vv])
            qh = q[t].float().view(G, rep, D)
            sc = torch.einsum("grd,ngd->grn", qh, K) * scale               # [G, rep, n]
            if softcap > 0.0:
                sc = softcap * torch.tanh(sc / softcap)
            if bias_kind != BIAS_NONE:
                dist = (i - torch.arange(lo, i + 1))
                if bias_kind == BIAS_LOG:
                    bias = -bias_a.view(H, 1) * torch.log(1.0 + bias_b.view(H, 1) * dist.float())
                else:
                    bias = bias_a[:, dist.clamp(max=bias_a.shape[1] - 1)]
                sc = sc + bias.view(G, rep, -1)
            if sink is not None:
                sc = torch.cat([sc, sink.view(G, rep, 1)], -1)
            p = torch.softmax(sc, -1)[..., : K.shape[0]]
            o = torch.einsum("grn,ngv->grv", p, Vv).reshape(1, H, V)
            if v_freq is not None:
                o = _rope_pairs(o, torch.tensor([-float(i)]), v_freq, 2 * v_freq.numel())
            o = o.reshape(H * V)
            if gate is not None:
                o = o * torch.sigmoid(gate[t].float())
            out[t] = o.to(out.dtype)


# ---------------------------------------------------------------------------------- linear attention
def linear_attn(q, k, v, g, z, head_decay, tau: float, q_scale: float, in_silu: bool, nw, norm_all: bool,
                gate_silu: bool, state, state_slots, context_lens, query_start, out, eps: float,
                num_seqs: int | None = None, cols_per_lane: int = 0, k_scale: float = 1.0, positions=None, inv_freq=None,
                rot_dims: int = 0, rot_half: bool = True, decay_exp: bool = False, bonus=None, norm_full: bool = False) -> None:
    """Decayed outer-product recurrence over state slots, state [slots, H, D, V] fp32:
        S <- diag(a_t) S + k_t v_t^T,  o_t = S^T (q_scale q_t)
    a_t = sigmoid(z_t)^(1 / tau) per key channel (``z`` fp32 [T, H * D]) or the constant head_decay[h];
    ``in_silu``: silu on q, k, v. With ``rot_dims`` > 0 the first rot_dims entries of every q / k head are
    turned by position * inv_freq (``rot_half``: entry i with i + rot_dims / 2, else 2i with 2i + 1), then k is
    multiplied by ``k_scale``. Then RMS norm of o (``nw`` None: no weight) (per head with a [V] weight, or with ``norm_all`` over
    the concatenated heads with a [H * V] weight), times silu(g) or sigmoid(g). A portion that starts at
    position 0 starts from a zero state. ``cols_per_lane`` (GPU): value columns a lane of the scan keeps, 0 =
    chosen by the launch's size. ``decay_exp``: a_t = exp(-exp(z_t)) instead. ``bonus`` [H, D] fp32: the state is read
    BEFORE its update and the current token's own outer product enters the output through the bonus,
        o_t = (S_(t-1) + diag(bonus) k_t v_t^T)^T (q_scale q_t),  then  S_t = diag(a_t) S_(t-1) + k_t v_t^T.
    ``norm_full`` (per-head norm): the weight is [H * V], one entry per output channel."""
    if q.is_cuda:
        H, D, V = state.shape[1], state.shape[2], state.shape[3]
        n = _C().linear_attn_scratch(q.shape[0], state_slots.numel(), H, D, V)
        scratch = torch.empty(n, dtype=torch.float32, device=q.device)
        _C().linear_attn(q, k, v, g, z, head_decay, tau, q_scale, in_silu, nw, norm_all, gate_silu, state, state_slots,
                         context_lens, query_start, out, eps, scratch, cols_per_lane, k_scale, positions, inv_freq,
                         rot_dims, rot_half, decay_exp, bonus, norm_full)
        return
    H, D, V = state.shape[1], state.shape[2], state.shape[3]
    S = state_slots.numel() if num_seqs is None else num_seqs
    act = torch.nn.functional.silu if in_silu else (lambda x: x)
    for s in range(S):
        t0, t1 = int(query_start[s]), int(query_start[s + 1])
        slot = int(state_slots[s])
        if t1 <= t0 or slot < 0:
            continue
        n = t1 - t0
        pos0 = int(context_lens[s]) - n
        St = state[slot].clone() if pos0 > 0 else torch.zeros(H, D, V)
        qq = act(q[t0:t1].float()).view(n, H, D)
        kk = act(k[t0:t1].float()).view(n, H, D)
        if rot_dims:
            turn = _rope_halves if rot_half else _rope_pairs
            qq, kk = turn(qq, positions[t0:t1], inv_freq, rot_dims), turn(kk, positions[t0:t1], inv_freq, rot_dims)
        qq, kk = qq * q_scale, kk * k_scale
        vv = act(v[t0:t1].float()).view(n, H, V)
        if z is not None and decay_exp:
            a = torch.exp(-torch.exp(z[t0:t1].float())).view(n, H, D)
        elif z is not None:
            a = torch.exp(torch.nn.functional.logsigmoid(z[t0:t1].float()) / tau).view(n, H, D)
        else:
            a = head_decay.view(1, H, 1).expand(n, H, D)
        o = torch.empty(n, H, V)
        for i in range(n):
            kv = kk[i][:, :, None] * vv[i][:, None, :]
            if bonus is not None:
                o[i] = torch.einsum("hdv,hd->hv", St + bonus[:, :, None] * kv, qq[i])
            St = a[i][:, :, None] * St + kv
            if bonus is None:
                o[i] = torch.einsum("hdv,hd->hv", St, qq[i])
        state[slot] = St
        one = 1.0 if nw is None else (nw.view(H, V) if norm_full else nw)
        if norm_all:
            of = o.reshape(n, H * V)
            of = of * (1.0 / torch.sqrt(of.pow(2).mean(-1, keepdim=True) + eps)) * one
        else:
            of = (o * (1.0 / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps)) * one).reshape(n, H * V)
        gg = g[t0:t1].float()
        of = of * (torch.nn.functional.silu(gg) if gate_silu else torch.sigmoid(gg))
        out[t0:t1] = of.to(out.dtype)
