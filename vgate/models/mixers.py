"""Token mixers and feed-forwards of layered hybrid models, one class per mechanism.

A mixer reads the layer's normed input ``h`` through rows of the layer's fused input projection
(``in_rows``: every matrix that multiplies ``h`` is stacked into one GEMM by the model) and owns
the rest of its weights. Constants of a mechanism are constructor parameters read from the layer's
spec, so another design can reuse a mixer with other values.

* :class:`LatentAttention` — attention through a low-rank key/value latent with one rotated key part
  shared by all heads; only the latent and that part are cached (paged), the per-head up-projections
  are absorbed into the query and the output.
* :class:`GeneralDelta` — generalized delta rule with per-channel decay over an fp32 state matrix
  per head, kept in a state slot per sequence.
* :class:`WindowAttention` — grouped-query attention over a sliding window (or all) of a paged key/value
  cache, optionally with one mean key / value per block of tokens that has left the window, a sink in the
  softmax denominator, query / key norms over the head or the whole projection, values rotated by
  their position, a bias on the scores that depends on the distance (logarithmic penalty or a learned
  table over distance buckets), per-head and per-position query temperatures, a sigmoid output gate.
* :class:`LinearAttention` — decayed outer-product recurrence S <- diag(a) S + k v^T, o = S^T q over an
  fp32 state per head in a state slot; the decay is a constant per head or a gated value per key channel;
  optional rotary positions on q / k.
* :class:`ShiftedLinearAttention` — the same kind of recurrence read before its update, with a bonus on the
  current token's own outer product, a decay exp(-exp(.)) per key channel from a low-rank gate, and every
  projection reading its own blend of the token's and the previous token's input (which is part of the state).
* :class:`ParallelMixers` — two mixers reading the same input, their outputs added with fixed scales.
* :class:`DenseFF`, :class:`MoEFF` — gated feed-forward; mixture of gated experts (sigmoid scores with a
  selection-only correction or softmax scores, clamped or SiLU experts, optional shared expert).
"""
from __future__ import annotations

import math
import os

import torch

from vgate import ops
from vgate.ops import seq

# bf16 matrices in the shape range the fragment-packed MFMA GEMMs are exercised on (N and K multiples
# of 64, K >= 512: the transformer families' projections) run there; the rest (and every fp32 matrix)
# through the row-major GEMM. "0" sends everything through the row-major one.
USE_PACKED = os.environ.get("VGATE_HYBRID_PACKED", "1") == "1"
PACKED_MIN_K = 512
# bf16 window attention on the MFMA kernel (keeps a transposed copy of the values); "0": the FMA kernel
USE_WINDOW_MFMA = os.environ.get("VGATE_WINDOW_MFMA", "1") == "1"


class Proj:
    """y = x W^T for a [N, K] matrix, on whichever GEMM takes its shape and dtype."""

    def __init__(self, w: torch.Tensor, device, f32: bool, silu_pair: bool = False, allow_packed: bool = True,
                 bias: torch.Tensor | None = None, pair_act: int = seq.ACT_SILU_MUL, limit: float = 0.0,
                 alpha: float = 1.702):
        N, K = w.shape
        self.N, self.K, self.f32, self.silu_pair = N, K, f32, silu_pair
        self.pair_act, self.limit, self.alpha = pair_act, limit, alpha
        dev = torch.device(device)
        n_ok = (N // 2) % 64 == 0 if silu_pair else N % 64 == 0
        self.packed = (USE_PACKED and allow_packed and not f32 and dev.type == "cuda" and n_ok and K % 64 == 0
                       and K >= PACKED_MIN_K)
        # the packed kernels' pair epilogue is SiLU: another pair activation runs the stacked [gate; up]
        # matrix as a plain packed GEMM and applies act(gate) * up in a row kernel
        self.split_act = self.packed and silu_pair and pair_act != seq.ACT_SILU_MUL
        self.bias = None
        if self.packed:
            self.lin = ops.Linear(w.to(dev, torch.bfloat16), kind="silu" if silu_pair and not self.split_act else "plain",
                                  bias=None if bias is None else bias.to(dev, torch.bfloat16).contiguous())
            self.w = None
        else:
            self.lin = None
            self.w = w.to(dev, torch.float32 if f32 else torch.bfloat16).contiguous()
            self.bias = None if bias is None else bias.to(dev, torch.float32).contiguous()
        self.out_features = N // 2 if silu_pair else N

    def nbytes(self) -> int:
        return self.lin.nbytes() if self.packed else self.w.numel() * self.w.element_size()

    def __call__(self, x: torch.Tensor, out_f32: bool = False, act: int = 0, out: torch.Tensor | None = None) -> torch.Tensor:
        M = x.shape[0]
        if self.split_act:
            if out is None:
                out = torch.empty(M, self.out_features, dtype=torch.bfloat16, device=x.device)
            return seq.glu_rows(ops.linear(x, self.lin), out, self.pair_act, limit=self.limit, alpha=self.alpha)
        if self.packed and act == 0:
            return ops.linear(x, self.lin, out=out, out_f32=out_f32)
        dt = torch.float32 if (out_f32 or self.f32) else torch.bfloat16
        if out is None:
            out = torch.empty(M, self.out_features, dtype=dt, device=x.device)
        if self.silu_pair:
            I = self.N // 2
            return seq.gemm(x, self.w[:I], out, w2=self.w[I:], act=self.pair_act, limit=self.limit, alpha=self.alpha)
        return seq.gemm(x, self.w, out, act=act, bias=self.bias)


def _f32(t: torch.Tensor, device) -> torch.Tensor:
    return t.to(device, torch.float32).contiguous()


def _pad8(w: torch.Tensor) -> torch.Tensor:
    """Zero rows up to a multiple of 8, so every segment of a fused projection starts 16-B aligned."""
    n = (-w.shape[0]) % 8
    return torch.cat([w, torch.zeros(n, w.shape[1], dtype=w.dtype)]) if n else w


# ------------------------------------------------------------------------------------------ mixers
class LatentAttention:
    """Attention through a low-rank key/value latent. spec: heads, dim, vdim, kv_rank, q_rank, scale, ``rot_dim``
    (size of the rotated key part all heads share; 0: none) with ``rot`` {dims, base}, and the options ``window``
    (position i sees j with 0 <= i - j < window; None: every earlier position), ``sink`` (one learned logit per
    head, tensor ``sink``, that only enters the softmax denominator), ``out_f32`` (the output projection writes
    fp32 for an fp32 residual sum)."""
    kind = "latent_attention"
    cache = "paged"
    TENSORS = ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o")
    FULL = 1 << 30

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool):
        m = spec
        self.H, self.D, self.R, self.V = int(m["heads"]), int(m["dim"]), int(m.get("rot_dim", 0)), int(m["vdim"])
        self.KR, self.QR = int(m["kv_rank"]), int(m["q_rank"])
        self.scale = float(m["scale"])
        self.window = self.FULL if m.get("window") is None else int(m["window"])
        if not 1 <= self.window <= self.FULL:
            raise ValueError("latent_attention: window >= 1")
        self.out_f32 = bool(m.get("out_f32", False))
        rot = m.get("rot") or {}
        dims = int(rot.get("dims", self.R))
        if dims > self.R or dims < 0:
            raise ValueError("latent_attention: rot.dims must be <= rot_dim")
        self.rot_dims = 2 * (dims // 2)  # entries in rotated pairs (an odd last one passes unchanged)
        self.eps = eps
        self.f32 = f32
        dev = torch.device(device)
        H, D, R, V, KR = self.H, self.D, self.R, self.V, self.KR
        self.inv_freq = seq.rope_inv_freq(dims, float(rot.get("base", 10000.0)), dev)  # base^(-2i / dims)
        self.in_rows = [("dq", tensors["dq"]), ("dkv", tensors["dkv"]), ("g", tensors["g"])]
        self.in_bias = {}
        self.dq_norm, self.dkv_norm = _f32(tensors["dq.norm"], dev), _f32(tensors["dkv.norm"], dev)
        self.uq = Proj(tensors["uq"], dev, f32)
        dt = torch.float32 if f32 else torch.bfloat16
        # absorbed up-projections, one matrix per head: q' = q_h W_uk[h] ([KR, D] as the GEMM's W), out = ol W_uv[h]^T
        self.uk_t = tensors["uk"].view(H, D, KR).transpose(1, 2).contiguous().to(dev, dt)
        self.uv = tensors["uv"].view(H, V, KR).contiguous().to(dev, dt)
        self.sink = _f32(tensors["sink"], dev) if m.get("sink") else None
        self.o = Proj(tensors["o"], dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        H, D, R, V = spec["heads"], spec["dim"], spec.get("rot_dim", 0), spec["vdim"]
        KR, QR = spec["kv_rank"], spec["q_rank"]
        out = {"dq": (QR, width), "dq.norm": (QR,), "uq": (H * (D + R), QR), "dkv": (KR + R, width),
               "dkv.norm": (KR,), "uk": (H * D, KR), "uv": (H * V, KR), "g": (H * V, width), "o": (width, H * V)}
        if spec.get("sink"):
            out["sink"] = (H,)
        return out

    def cache_shape(self, num_blocks: int, block_size: int, num_slots: int) -> tuple:
        """One flat buffer per layer: rows [blocks, page, kv_rank + rot_dim], then (bf16) the transposed copy of
        the latent part [blocks, kv_rank, page] that the MFMA attention kernel reads."""
        self._page = block_size
        return (num_blocks * block_size * (self.KR + self.R + (0 if self.f32 else self.KR)),)

    def _views(self, cache: torch.Tensor):
        E, block_size = self.KR + self.R, getattr(self, "_page", 16)
        per = block_size * (E + (0 if self.f32 else self.KR))
        nb = cache.numel() // per
        rows = cache[: nb * block_size * E].view(nb, block_size, E)
        tr = None if self.f32 else cache[nb * block_size * E:].view(nb, self.KR, block_size)
        return rows, tr

    def cache_dtype(self):
        return torch.float32 if self.f32 else torch.bfloat16

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, device) -> torch.Tensor:
        return torch.zeros(self.cache_shape(num_blocks, block_size, num_slots), dtype=self.cache_dtype(), device=device)

    def page_bytes(self, block_size: int) -> int:
        return math.prod(self.cache_shape(1, block_size, 1)) * (4 if self.f32 else 2)

    def nbytes(self) -> int:
        return self.uq.nbytes() + self.o.nbytes() + 2 * self.uk_t.numel() * self.uk_t.element_size()

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        H, D, R, V, KR = self.H, self.D, self.R, self.V, self.KR
        E = KR + R
        dt, dev = h.dtype, h.device
        cq = torch.empty(T, self.QR, dtype=dt, device=dev)
        seq.norm_rows(cols(P, "dq"), self.dq_norm, self.eps, cq)
        q = self.uq(cq)
        cache, cache_t = self._views(cache)
        seq.latent_write(cols(P, "dkv"), self.dkv_norm, self.eps, sv.positions, sv.slots, self.inv_freq,
                         self.rot_dims, cache, KR, cache_t=cache_t)
        qa = torch.empty(T, H, E, dtype=dt, device=dev)
        seq.gemm(q.view(T, H, D + R)[:, :, :D].permute(1, 0, 2), self.uk_t, qa[:, :, :KR].permute(1, 0, 2))
        if R:
            seq.latent_qrope(q, sv.positions, self.inv_freq, self.rot_dims, qa, H, D, KR, R)
        ol = torch.empty(T, H, KR, dtype=dt, device=dev)
        seq.latent_attn(qa, cache, sv.block_tables, sv.context_lens, sv.query_start, ol, self.scale, H, KR, R,
                        num_seqs=sv.num_seqs or None, cache_t=cache_t, window=self.window, sink=self.sink)
        og = torch.empty(T, H, V, dtype=dt, device=dev)
        gate = cols(P, "g").unflatten(1, (H, V)).permute(1, 0, 2)
        seq.gemm(ol.permute(1, 0, 2), self.uv, og.permute(1, 0, 2), gate=gate)
        return self.o(og.view(T, H * V), out_f32=self.out_f32)


class GeneralDelta:
    kind = "general_delta"
    cache = "state"
    TENSORS = ("r", "k", "v", "g", "a", "a.b", "w1", "w2", "w0", "norm", "o")
    DECAY_C = math.exp(-0.5)   # w = exp(-DECAY_C * sigmoid(.))
    UNIT_EPS = 1e-6            # u = k / sqrt(sum(k^2) + UNIT_EPS)

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool,
                 decay_c: float | None = None, unit_eps: float | None = None):
        self.H, self.D = int(spec["heads"]), int(spec["dim"])
        if self.D > 128:
            raise ValueError("general_delta: the recurrence kernel keeps a state column in registers: head size <= 128")
        self.eps, self.f32 = eps, f32
        self.decay_c = self.DECAY_C if decay_c is None else decay_c
        self.unit_eps = self.UNIT_EPS if unit_eps is None else unit_eps
        dev = torch.device(device)
        self.in_rows = [(n, tensors[n]) for n in ("r", "k", "v", "g", "a")]
        self.in_bias = {}
        if tensors["w2"].shape[1] != tensors["w1"].shape[0]:
            raise ValueError("general_delta: w1 / w2 disagree on the decay's width")
        self.w1 = Proj(tensors["w1"], dev, f32, allow_packed=False)  # tanh in its epilogue
        self.w2 = Proj(tensors["w2"], dev, f32)
        self.w0, self.ab, self.nw = _f32(tensors["w0"], dev), _f32(tensors["a.b"], dev), _f32(tensors["norm"], dev)
        self.o = Proj(tensors["o"], dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        n = spec["heads"] * spec["dim"]
        # None: the decay's low-rank width, which only the checkpoint's tensors give
        return {"r": (n, width), "k": (n, width), "v": (n, width), "g": (n, width), "a": (n, width), "a.b": (n,),
                "w1": (None, width), "w2": (n, None), "w0": (n,), "norm": (n,), "o": (width, n)}

    def cache_shape(self, num_blocks: int, block_size: int, num_slots: int) -> tuple:
        return (num_slots, self.H, self.D, self.D)

    def cache_dtype(self):
        return torch.float32

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, device) -> torch.Tensor:
        return torch.zeros(self.cache_shape(num_blocks, block_size, num_slots), dtype=torch.float32, device=device)

    def page_bytes(self, block_size: int) -> int:
        return 0

    def nbytes(self) -> int:
        return self.w1.nbytes() + self.w2.nbytes() + self.o.nbytes()

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        wl = self.w2(self.w1(h, act=seq.ACT_TANH))
        out = torch.empty(T, self.H * self.D, dtype=h.dtype, device=h.device)
        seq.delta_rule(cols(P, "r"), cols(P, "k"), cols(P, "v"), cols(P, "g"), cols(P, "a"), wl, self.w0, self.ab,
                       self.nw, cache, sv.state_slots, sv.context_lens, sv.query_start, out, self.decay_c,
                       self.unit_eps, self.eps, num_seqs=sv.num_seqs or None)
        return self.o(out)


class WindowAttention:
    """Grouped-query attention over the last ``window`` positions of a paged key/value cache.

    spec: heads, kv_heads, dim, vdim, scale, rot {base, dims, scaling}, window, and the options
    ``pool`` (P > 0: every block of P tokens that lies wholly before the window is seen through the
    mean of its cached keys and the mean of its cached values; tokens between such a block and the
    window are not seen), ``qk_norm`` ("none" | "head": RMS norm per head with one [dim] weight |
    "all": one RMS norm over the whole projection with a [heads * dim] weight), ``rotate_values``
    (the cached value of position j is turned by j in pairs over all of vdim, the attention output
    of position i is turned back by i), ``sink`` (one learned logit per head that only enters the
    softmax denominator), ``bias`` (q / k / v biases), ``out_bias``.
    ``window`` None: every earlier position is seen. ``qk_norm_weight`` False: the head norm has no weight.
    ``head_temp``: the scores of head h are multiplied by the tensor ``temp`` [h]. ``q_temp`` {coef, every}:
    the query at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1). ``dist_bias``: a term
    of the score that depends on the head and the distance n = i - j alone, {"kind": "log"}:
    -r1[h] ln(1 + r2[h] n) (tensors ``r1``, ``r2``); {"kind": "table", "far": F}: rel[bucket(n), h] with the
    learned tensor ``rel`` [B, heads], bucket(n) = n below B/2 and log-spaced rows from B/2 to F above
    (:func:`distance_buckets`). ``gate`` "sigmoid": the heads' outputs are multiplied by sigmoid(W_g h)
    before the output projection. ``rot.layout`` "pairs" (entry 2i with 2i + 1, the default) or "half" (entry i
    with i + dims / 2). ``softcap`` c > 0: the scaled score s becomes c tanh(s / c).
    ``maps`` {count: 2, init: d}: every head has two query / key maps (q and k carry [map 1, map 2] per head,
    each of size dim) that are two attentions over the same values; with lam = exp(lq1 . lk1) - exp(lq2 . lk2) + d
    (tensors ``lq1`` .. ``lk2`` [dim], one number per layer) the head's output is (a1 - lam a2), divided by its
    root mean square over vdim, times (1 - d). Inside, the maps run as 2 heads query heads over 2 kv_heads key
    heads that share kv_heads value heads; the query rows are regrouped once at load so that the heads of one key
    head are contiguous.
    """
    kind = "window_attention"
    cache = "paged"
    FULL = 1 << 30   # "window" of a layer that sees every earlier position

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool):
        m = spec
        self.H, self.G, self.D, self.V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        if self.G < 1 or self.H % self.G:
            raise ValueError("window_attention: heads must be a multiple of kv_heads")
        self.scale, self.pool = float(m["scale"]), int(m.get("pool") or 0)
        self.window = self.FULL if m.get("window") is None else int(m["window"])
        if self.window < 1 or self.pool < 0 or self.window > self.FULL:
            raise ValueError("window_attention: window >= 1, pool >= 0")
        if self.pool and m.get("window") is None:
            raise ValueError("window_attention: pooled blocks need a window")
        self.qk_norm = m.get("qk_norm", "none")
        if self.qk_norm not in ("none", "head", "all"):
            raise ValueError(f"window_attention: qk_norm {self.qk_norm!r}")
        rot = m.get("rot") or {}
        dims = int(rot.get("dims", 0))
        if dims > self.D or dims < 0:
            raise ValueError("window_attention: rot.dims must be <= dim")
        self.rot_dims = 2 * (dims // 2)
        if rot.get("layout", "pairs") not in ("pairs", "half"):
            raise ValueError(f"window_attention: rot.layout {rot.get('layout')!r}")
        self.rot_half = rot.get("layout", "pairs") == "half"
        self.softcap = float(m.get("softcap") or 0.0)
        self.eps, self.f32 = eps, f32
        dev = torch.device(device)
        base = float(rot.get("base", 10000.0))
        self.inv_freq = seq.rope_inv_freq(dims, base, dev, scaling=rot.get("scaling"))
        self.v_freq = seq.rope_inv_freq(self.V, base, dev) if m.get("rotate_values") else None
        self.gated = m.get("gate") == "sigmoid"
        if m.get("gate") not in (None, "sigmoid"):
            raise ValueError(f"window_attention: gate {m.get('gate')!r}")
        maps = m.get("maps") or {}
        self.maps = int(maps.get("count", 1))
        if self.maps not in (1, 2):
            raise ValueError("window_attention: one or two score maps per head")
        # query / key heads the kernels see; the value heads stay kv_heads
        self.HQ, self.GK = self.H * self.maps, self.G * self.maps
        rep = self.H // self.G

        def regroup(t: torch.Tensor) -> torch.Tensor:
            """Rows of a per-query-head tensor [heads x maps x n, ...] -> (key/value head, map, head in group)."""
            if self.maps == 1:
                return t
            n = t.shape[0] // (self.H * 2)
            return t.reshape(self.G, rep, 2, n, *t.shape[1:]).transpose(1, 2).reshape(t.shape).contiguous()

        self.lam = self.out_scale = None
        if self.maps == 2:
            if self.pool or m.get("rotate_values") or m.get("head_temp") or m.get("dist_bias") or m.get("q_temp"):
                raise ValueError("window_attention: two score maps do not combine with pooled blocks, turned values, "
                                 "temperatures or distance terms")
            d = float(maps["init"])
            dot = lambda a, b: float((tensors[a].double() * tensors[b].double()).sum())  # noqa: E731
            self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + d
            self.out_scale = 1.0 - d
        self.in_rows = [("q", regroup(tensors["q"])), ("k", tensors["k"]), ("v", tensors["v"])]
        if self.gated:
            self.in_rows.append(("g", tensors["g"]))
        self.in_bias = {"q": regroup(tensors["q.b"]), "k": tensors["k.b"], "v": tensors["v.b"]} if m.get("bias") else {}
        self.qw = self.kw = None
        if self.qk_norm != "none":
            if m.get("qk_norm_weight", True):
                per_head = self.qk_norm == "head"
                self.qw = _f32(tensors["q.norm"] if per_head else regroup(tensors["q.norm"]), dev)
                self.kw = _f32(tensors["k.norm"], dev)
            else:   # a norm without a weight: ones
                per_head = self.qk_norm == "head"
                self.qw = torch.ones(self.D if per_head else self.HQ * self.D, dtype=torch.float32, device=dev)
                self.kw = torch.ones(self.D if per_head else self.GK * self.D, dtype=torch.float32, device=dev)
        self.sink = None
        if m.get("sink"):   # (with two maps: the head's sink in both)
            sk = tensors["sink"]
            self.sink = _f32(regroup(sk.repeat_interleave(2)) if self.maps == 2 else sk, dev)
        self.head_temp = _f32(tensors["temp"], dev) if m.get("head_temp") else None
        qt = m.get("q_temp") or {}
        self.q_temp = (float(qt.get("coef", 0.0)), int(qt.get("every", 1)))
        if self.q_temp[1] < 1:
            raise ValueError("window_attention: q_temp.every >= 1")
        db = m.get("dist_bias") or {}
        self.bias_kind, self.bias_a, self.bias_b = seq.BIAS_NONE, None, None
        if db.get("kind") == "log":
            self.bias_kind, self.bias_a, self.bias_b = seq.BIAS_LOG, _f32(tensors["r1"], dev), _f32(tensors["r2"], dev)
        elif db.get("kind") == "table":
            rel = tensors["rel"].float()
            rows = distance_buckets(rel.shape[0], float(db["far"]))
            # expanded once to one entry per distance (the last stands for every larger one), head-major
            self.bias_kind, self.bias_a = seq.BIAS_TABLE, rel[torch.tensor(rows)].t().contiguous().to(dev)
            if rel.shape[1] != self.H:
                raise ValueError("window_attention: the distance table needs one column per head")
        elif db:
            raise ValueError(f"window_attention: dist_bias kind {db.get('kind')!r}")
        if self.bias_kind and self.pool:
            raise ValueError("window_attention: a distance bias and pooled blocks do not combine")
        self.o = Proj(tensors["o"], dev, f32, bias=tensors["o.b"] if m.get("out_bias") else None)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
        mp = int((spec.get("maps") or {}).get("count", 1))
        out = {"q": (H * mp * D, width), "k": (G * mp * D, width), "v": (G * V, width), "o": (width, H * V)}
        if mp == 2:
            out.update({n: (D,) for n in ("lq1", "lk1", "lq2", "lk2")})
        if spec.get("bias"):
            out.update({"q.b": (H * mp * D,), "k.b": (G * mp * D,), "v.b": (G * V,)})
        weighted = spec.get("qk_norm_weight", True)
        if weighted and spec.get("qk_norm", "none") == "head":
            out.update({"q.norm": (D,), "k.norm": (D,)})
        elif weighted and spec.get("qk_norm") == "all":
            out.update({"q.norm": (H * mp * D,), "k.norm": (G * mp * D,)})
        if spec.get("gate"):
            out["g"] = (H * V, width)
        if spec.get("head_temp"):
            out["temp"] = (H,)
        kind = (spec.get("dist_bias") or {}).get("kind")
        if kind == "log":
            out.update({"r1": (H,), "r2": (H,)})
        elif kind == "table":   # None: the number of buckets, which only the tensor gives
            out["rel"] = (None, H)
        if spec.get("sink"):
            out["sink"] = (H,)
        if spec.get("out_bias"):
            out["o.b"] = (width,)
        return out

    def pooled_per_page(self, block_size: int) -> int:
        """Pooled rows a cache page carries: block b's means live in the page of its last position
        b P + P - 1, in row (that position mod page) / P."""
        return (block_size + self.pool - 1) // self.pool if self.pool else 0

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, device) -> tuple:
        dt = torch.float32 if self.f32 else torch.bfloat16
        npool = self.pooled_per_page(block_size)
        z = lambda heads, rows, d: torch.zeros(num_blocks, heads, rows, d, dtype=dt, device=device)  # noqa: E731
        # bf16 on the GPU: a second, transposed copy of the values for the MFMA kernel's weighted sum
        vt = torch.zeros(num_blocks, self.G, self.V, block_size, dtype=dt, device=device) if self._transposed(device) else None
        return (z(self.GK, block_size, self.D), z(self.G, block_size, self.V),
                z(self.G, npool, self.D) if npool else None, z(self.G, npool, self.V) if npool else None, vt)

    def _transposed(self, device) -> bool:
        return not self.f32 and torch.device(device).type == "cuda" and USE_WINDOW_MFMA

    def page_bytes(self, block_size: int) -> int:
        n = (block_size + self.pooled_per_page(block_size)) * (self.GK * self.D + self.G * self.V) * (4 if self.f32 else 2)
        return n + (0 if self.f32 else block_size * self.G * self.V * 2)

    def nbytes(self) -> int:
        return self.o.nbytes()

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        kc, vc, kp, vp, vt = cache
        q = torch.empty(T, self.HQ * self.D, dtype=h.dtype, device=h.device)
        seq.window_write(cols(P, "q"), cols(P, "k"), cols(P, "v"), self.qw, self.kw, self.eps, self.qk_norm == "all",
                         sv.positions, sv.slots, self.inv_freq, self.rot_dims, self.v_freq, kc, vc, q, self.HQ, self.GK, vt=vt,
                         q_head_scale=self.head_temp, q_temp_coef=self.q_temp[0], q_temp_every=self.q_temp[1],
                         rot_half=self.rot_half)
        if self.pool:
            seq.window_pool(kc, vc, kp, vp, sv.positions, sv.block_tables, sv.query_start, self.pool,
                            num_seqs=sv.num_seqs or None)
        gate = cols(P, "g") if self.gated else None
        o = torch.empty(T, self.HQ * self.V, dtype=h.dtype, device=h.device)
        seq.window_attn(q, kc, vc, kp, vp, sv.block_tables, sv.context_lens, sv.query_start, o, self.scale, self.HQ,
                        self.window, self.pool, self.sink, self.v_freq, num_seqs=sv.num_seqs or None, vt=vt,
                        bias_kind=self.bias_kind, bias_a=self.bias_a, bias_b=self.bias_b,
                        gate=gate if self.maps == 1 else None, softcap=self.softcap)
        if self.maps == 2:   # (a1 - lam a2) / rms * (1 - init) * sigmoid(gate), heads back in their own order
            both, o = o, torch.empty(T, self.H * self.V, dtype=h.dtype, device=h.device)
            seq.map_pair_combine(both, self.lam, self.out_scale, self.eps, gate, o, self.H, self.G, self.V)
        return self.o(o, out_f32=True)


def distance_buckets(B: int, far: float) -> list:
    """Row of a [B, heads] distance table for every distance 0 .. ceil(far): distances below B // 2 have a
    row each, the rows from B // 2 on are spaced evenly in ln(distance) between B // 2 and ``far``, and the
    last row takes everything beyond (so the list's last entry stands for all larger distances)."""
    half = B // 2
    if half < 1 or far <= half:
        raise ValueError("distance table: at least two rows, and far > rows / 2")
    rows = []
    for n in range(max(int(math.ceil(far)), half) + 1):
        rows.append(n if n < half else
                    min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half)))))
    return rows


class LinearAttention:
    """Decayed outer-product recurrence per head over an fp32 state [dim, vdim] in a state slot:
    S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T (q_scale q_t).

    spec: heads, dim, vdim, ``decay`` ({"kind": "head", "values": [one constant per head]} or
    {"kind": "channel", "tau": tau}: a = sigmoid(z)^(1 / tau) per key channel with z = W_a2 (W_a1 h) +
    b, a low-rank gate whose width the checkpoint's tensors give), ``q_scale``, ``in_act`` ("none" |
    "silu" on q, k and v), ``out_norm`` ("head": RMS norm per head with one [vdim] weight | "all":
    over the concatenated heads with a [heads * vdim] weight; ``norm_weight`` False: no weight),
    ``gate_act`` ("silu" | "sigmoid" of W_g h, multiplied onto the normed output before the output
    projection), ``rot`` {dims, base, layout "half" | "pairs"}: rotary positions on the first ``dims``
    entries of every q / k head (entry i paired with i + dims / 2, or 2i with 2i + 1), ``k_scale``
    (keys multiplied after the rotation).
    """
    kind = "linear_attention"
    cache = "state"

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool):
        self.H, self.D, self.V = int(spec["heads"]), int(spec["dim"]), int(spec["vdim"])
        if self.D > seq.LINEAR_ATTN_MAX_DIM:
            raise ValueError(f"linear_attention: the recurrence keeps a state column in registers: dim <= {seq.LINEAR_ATTN_MAX_DIM}")
        self.eps, self.f32 = eps, f32
        dev = torch.device(device)
        dec = spec["decay"]
        self.channel = dec["kind"] == "channel"
        if dec["kind"] not in ("channel", "head"):
            raise ValueError(f"linear_attention: decay kind {dec['kind']!r}")
        for key, allowed in (("in_act", ("none", "silu")), ("out_norm", ("head", "all")), ("gate_act", ("silu", "sigmoid"))):
            if spec[key] not in allowed:
                raise ValueError(f"linear_attention: {key} {spec[key]!r}")
        self.q_scale, self.k_scale = float(spec.get("q_scale", 1.0)), float(spec.get("k_scale", 1.0))
        rot = spec.get("rot") or {}
        dims = int(rot.get("dims", 0))
        if dims > self.D or dims < 0 or rot.get("layout", "half") not in ("half", "pairs"):
            raise ValueError("linear_attention: rot.dims <= dim, layout half | pairs")
        self.rot_dims, self.rot_half = 2 * (dims // 2), rot.get("layout", "half") == "half"
        self.inv_freq = seq.rope_inv_freq(dims, float(rot.get("base", 10000.0)), dev) if self.rot_dims else None
        self.in_silu, self.norm_all, self.gate_silu = spec["in_act"] == "silu", spec["out_norm"] == "all", spec["gate_act"] == "silu"
        self.in_rows = [(n, tensors[n]) for n in ("q", "k", "v", "g")]
        self.in_bias = {}
        self.tau, self.a2, self.head_decay = 1.0, None, None
        if self.channel:
            self.tau = float(dec["tau"])
            if tensors["a2"].shape[1] != tensors["a1"].shape[0]:
                raise ValueError("linear_attention: a1 / a2 disagree on the gate's width")
            self.in_rows.append(("a1", tensors["a1"]))
            self.a2 = Proj(tensors["a2"], dev, f32, allow_packed=False, bias=tensors["a2.b"])  # fp32 gate logits
        else:
            self.head_decay = torch.tensor([float(d) for d in dec["values"]], dtype=torch.float32, device=dev)
        self.nw = _f32(tensors["norm"], dev) if spec.get("norm_weight", True) else None
        self.o = Proj(tensors["o"], dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        H, D, V = spec["heads"], spec["dim"], spec["vdim"]
        out = {"q": (H * D, width), "k": (H * D, width), "v": (H * V, width), "g": (H * V, width), "o": (width, H * V)}
        if spec.get("norm_weight", True):
            out["norm"] = (H * V,) if spec["out_norm"] == "all" else (V,)
        if spec["decay"]["kind"] == "channel":  # None: the gate's width, which only the tensors give
            out.update({"a1": (None, width), "a2": (H * D, None), "a2.b": (H * D,)})
        return out

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, device) -> torch.Tensor:
        return torch.zeros(num_slots, self.H, self.D, self.V, dtype=torch.float32, device=device)

    def page_bytes(self, block_size: int) -> int:
        return 0

    def nbytes(self) -> int:
        return self.o.nbytes() + (self.a2.nbytes() if self.a2 else 0)

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        z = self.a2(cols(P, "a1"), out_f32=True) if self.channel else None
        out = torch.empty(T, self.H * self.V, dtype=h.dtype, device=h.device)
        seq.linear_attn(cols(P, "q"), cols(P, "k"), cols(P, "v"), cols(P, "g"), z, self.head_decay, self.tau, self.q_scale,
                        self.in_silu, self.nw, self.norm_all, self.gate_silu, cache, sv.state_slots, sv.context_lens,
                        sv.query_start, out, self.eps, num_seqs=sv.num_seqs or None, k_scale=self.k_scale,
                        positions=sv.positions, inv_freq=self.inv_freq, rot_dims=self.rot_dims, rot_half=self.rot_half)
        return self.o(out, out_f32=True)


class ShiftedLinearAttention:
    """Decayed outer-product recurrence per head that is read BEFORE its update, with a bonus on the current
    token's own outer product, over an fp32 state [dim, dim] per head in a state slot:
        o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,   S_t = diag(w_t) S_(t-1) + k_t v_t^T
    w_t = exp(-exp(W_w2 tanh(W_w1 x_w) + w0)) per head and key channel (fp32; the gate's low-rank width is the
    tensors'). Each of r, k, v, g, w reads its own blend x_s = h + (h' - h) mu_s of the token's input h and the
    previous token's h' (zeros before the first token; the last token's h is kept in the state slot beside S).
    Output: every head's o divided by its root mean square, the heads concatenated, times ``norm`` [heads * dim],
    times silu(W_g x_g), then W_o. spec: heads, dim."""
    kind = "wkv"
    cache = "state"
    SHIFTS = ("r", "k", "v", "g", "w")

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool):
        self.H, self.D = int(spec["heads"]), int(spec["dim"])
        if self.D > seq.LINEAR_ATTN_MAX_DIM:
            raise ValueError(f"wkv: the recurrence keeps a state column in registers: dim <= {seq.LINEAR_ATTN_MAX_DIM}")
        self.eps, self.f32, self.W = eps, f32, width
        dev = torch.device(device)
        self.in_rows, self.in_bias = [], {}   # nothing reads the layer's input itself
        self.mu = torch.stack([tensors["mu." + n].float() for n in self.SHIFTS]).to(dev).contiguous()
        self.r, self.k, self.v, self.g = (Proj(tensors[n], dev, f32) for n in ("r", "k", "v", "g"))
        if tensors["w2"].shape[1] != tensors["w1"].shape[0]:
            raise ValueError("wkv: w1 / w2 disagree on the decay gate's width")
        self.w1 = Proj(tensors["w1"], dev, f32, allow_packed=False)                      # tanh in its epilogue
        self.w2 = Proj(tensors["w2"], dev, f32, allow_packed=False, bias=tensors["w0"])  # fp32 logits + w0
        self.u = _f32(tensors["u"].reshape(self.H, self.D), dev)
        self.nw = _f32(tensors["norm"], dev)
        self.o = Proj(tensors["o"], dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        H, D = spec["heads"], spec["dim"]
        n = H * D
        out = {"mu." + s: (width,) for s in ShiftedLinearAttention.SHIFTS}
        out.update({"r": (n, width), "k": (n, width), "v": (n, width), "g": (n, width), "w1": (None, width), "w2": (n, None),
                    "w0": (n,), "u": (H, D), "norm": (n,), "o": (width, n)})
        return out

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, device) -> tuple:
        """(the recurrence's state, the last token's input) per state slot."""
        return (torch.zeros(num_slots, self.H, self.D, self.D, dtype=torch.float32, device=device),
                torch.zeros(num_slots, self.W, dtype=torch.float32, device=device))

    def page_bytes(self, block_size: int) -> int:
        return 0

    def nbytes(self) -> int:
        return sum(p.nbytes() for p in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.o))

    def forward(self, h, P, cols, sv, cache) -> torch.Tensor:
        T = h.shape[0]
        state, last = cache
        x = torch.empty(len(self.SHIFTS), T, self.W, dtype=h.dtype, device=h.device)
        seq.shift_mix(h, last, self.mu, sv.state_slots, sv.context_lens, sv.query_start, x, num_seqs=sv.num_seqs or None)
        r, k, v, g = self.r(x[0]), self.k(x[1]), self.v(x[2]), self.g(x[3])
        z = self.w2(self.w1(x[4], act=seq.ACT_TANH), out_f32=True)
        out = torch.empty(T, self.H * self.D, dtype=h.dtype, device=h.device)
        seq.linear_attn(r, k, v, g, z, None, 1.0, 1.0, False, self.nw, False, True, state, sv.state_slots, sv.context_lens,
                        sv.query_start, out, self.eps, num_seqs=sv.num_seqs or None, decay_exp=True, bonus=self.u,
                        norm_full=True)
        return self.o(out, out_f32=True)


class ParallelMixers:
    """Two mixers side by side on the same input: y = left_scale * left(h) + right_scale * right(h).
    spec: ``left`` / ``right`` = (key of MIXERS, that mixer's spec); tensors under ``left.`` / ``right.``.
    ``forward`` returns the two outputs with their scales; the layer's residual kernel adds them."""
    kind = "parallel"
    cache = "both"

    def __init__(self, spec: dict, width: int, eps: float, tensors: dict, device, f32: bool):
        self.parts, self.scales = [], (float(spec["left_scale"]), float(spec["right_scale"]))
        self.in_rows, self.in_bias = [], {}
        for side in ("left", "right"):
            kind, sub_spec = spec[side]
            t = {k[len(side) + 1:]: v for k, v in tensors.items() if k.startswith(side + ".")}
            mx = MIXERS[kind](sub_spec, width, eps, t, device, f32)
            self.in_rows += [(f"{side}.{n}", w) for n, w in mx.in_rows]
            self.in_bias.update({f"{side}.{n}": b for n, b in mx.in_bias.items()})
            del mx.in_rows
            self.parts.append((side, mx))

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        out = {}
        for side in ("left", "right"):
            kind, sub_spec = spec[side]
            out.update({f"{side}.{k}": v for k, v in MIXERS[kind].shapes(sub_spec, width).items()})
        return out

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, device) -> tuple:
        return tuple(mx.allocate(num_blocks, block_size, num_slots, device) for _, mx in self.parts)

    def page_bytes(self, block_size: int) -> int:
        return sum(mx.page_bytes(block_size) for _, mx in self.parts)

    def nbytes(self) -> int:
        return sum(mx.nbytes() for _, mx in self.parts)

    def forward(self, h, P, cols, sv, cache) -> tuple:
        ys = [mx.forward(h, P, (lambda P_, n, s=side: cols(P_, f"{s}.{n}")), sv, c)
              for (side, mx), c in zip(self.parts, cache)]
        return ys[0], self.scales[0], ys[1], self.scales[1]


MIXERS = {c.kind: c for c in (LatentAttention, GeneralDelta, WindowAttention, LinearAttention, ShiftedLinearAttention,
                              ParallelMixers)}


# ------------------------------------------------------------------------------------ feed-forwards
class DenseFF:
    """down(act(gate h) * (up h)); spec ``act``: "silu" (default), "gelu_tanh", or "clamped" with ``limit`` L:
    g = min(gate h, L), u = clamp(up h, -L, L), down(g * sigmoid(ALPHA g) * (u + 1))."""
    ACTS = {"silu": seq.ACT_SILU_MUL, "gelu_tanh": seq.ACT_GELU_TANH_MUL, "clamped": seq.ACT_CLAMPED_GLU}
    ALPHA = 1.702

    def __init__(self, spec: dict, width: int, tensors: dict, device, f32: bool):
        act = spec.get("act", "silu")
        if act not in self.ACTS:
            raise ValueError(f"dense feed-forward: act {act!r}")
        self.gate_up = Proj(torch.cat([tensors["gate"], tensors["up"]]), device, f32, silu_pair=True,
                            pair_act=self.ACTS[act], limit=float(spec.get("limit", 0.0)), alpha=self.ALPHA)
        self.down = Proj(tensors["down"], device, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        return {"gate": (spec["ff"], width), "up": (spec["ff"], width), "down": (width, spec["ff"])}

    def nbytes(self) -> int:
        return self.gate_up.nbytes() + self.down.nbytes()

    def forward(self, h: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
        return self.down(self.gate_up(h), out_f32=out_f32)


class MoEFF:
    """Routed experts: scores s = sigmoid(z) or softmax(z) over all experts (``router.score``, fp32); the
    ``top`` largest of s (+ a selection-only ``correction`` tensor unless ``router.correction`` is False)
    are chosen, weighted by their scores over the chosen scores' sum, times ``router.scale``. Expert
    (``expert.act``): "clamped": g = min(gate h, L), u = clamp(up h, -L, L), down(g * sigmoid(alpha g) * (u + 1));
    "silu": down(silu(gate h) * (up h)). ``shared`` {ff}: a dense gated expert every token runs, added."""
    ALPHA = 1.702
    SUM_EPS = 1e-20

    def __init__(self, spec: dict, width: int, tensors: dict, device, f32: bool):
        r = spec["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        self.ff = int(spec["expert"]["ff"])
        self.act = {"clamped": seq.ACT_CLAMPED_GLU, "silu": seq.ACT_SILU_MUL}[spec["expert"].get("act", "clamped")]
        self.limit = float(spec["expert"]["limit"]) if self.act == seq.ACT_CLAMPED_GLU else 0.0
        self.softmax = {"sigmoid": False, "softmax": True}[r.get("score", "sigmoid")]
        self.scale = float(r.get("scale", 1.0))
        dev = torch.device(device)
        dt = torch.float32 if f32 else torch.bfloat16
        self.f32 = f32
        self.router = Proj(tensors["router"], dev, f32, allow_packed=False)  # fp32 logits, N = experts
        self.corr = _f32(tensors["correction"], dev) if r.get("correction", True) else None
        st = lambda n: torch.stack([tensors[f"e{e}.{n}"] for e in range(self.E)]).to(dev, dt).contiguous()  # noqa: E731
        self.gate, self.up, self.down = st("gate"), st("up"), st("down")
        self.shared = None
        if spec.get("shared"):
            sh = {k[len("shared."):]: v for k, v in tensors.items() if k.startswith("shared.")}
            self.shared = DenseFF({"ff": int(spec["shared"]["ff"]), "act": spec["shared"].get("act", "silu")}, width, sh, dev, f32)

    @staticmethod
    def shapes(spec: dict, width: int) -> dict:
        E, ff = spec["router"]["experts"], spec["expert"]["ff"]
        out = {"router": (E, width)}
        if spec["router"].get("correction", True):
            out["correction"] = (E,)
        for e in range(E):
            out.update({f"e{e}.gate": (ff, width), f"e{e}.up": (ff, width), f"e{e}.down": (width, ff)})
        if spec.get("shared"):
            out.update({"shared." + k: v for k, v in DenseFF.shapes(spec["shared"], width).items()})
        return out

    def nbytes(self) -> int:
        return (self.router.nbytes() + 3 * self.gate.numel() * self.gate.element_size()
                + (self.shared.nbytes() if self.shared else 0))

    def forward(self, h: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
        T, W = h.shape
        dev, dt = h.device, h.dtype
        z = self.router(h, out_f32=True)
        idx = torch.empty(T, self.top, dtype=torch.int32, device=dev)
        wts = torch.empty(T, self.top, dtype=torch.float32, device=dev)
        seq.moe_route(z, self.corr, self.top, self.SUM_EPS, idx, wts, softmax=self.softmax, scale=self.scale)
        rows = torch.empty(T * self.top, dtype=torch.int32, device=dev)
        pos = torch.empty(T * self.top, dtype=torch.int32, device=dev)
        off = torch.empty(self.E + 1, dtype=torch.int32, device=dev)
        seq.moe_sort(idx, self.E, rows, pos, off)
        a1 = torch.empty(T * self.top, self.ff, dtype=dt, device=dev)
        seq.gemm(h, self.gate, a1, w2=self.up, a_rows=rows, group_off=off, act=self.act, limit=self.limit,
                 alpha=self.ALPHA)
        y = torch.empty(T * self.top, W, dtype=dt, device=dev)
        seq.gemm(a1, self.down, y, group_off=off)
        out = torch.empty(T, W, dtype=torch.float32 if out_f32 else dt, device=dev)
        seq.moe_combine(y, pos, wts, out, add=self.shared.forward(h, out_f32=out_f32) if self.shared else None)
        return out


FEED_FORWARDS = {"dense": DenseFF, "moe": MoEFF}
