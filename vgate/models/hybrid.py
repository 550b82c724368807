"""Layered hybrid decoder: a list of layers, each a token mixer (``vgate.models.mixers.MIXERS``) and
an optional feed-forward, over an fp32 residual stream.

One forward pass = one engine step over a flat token batch (any mix of prompt portions and single
decoded tokens) with all step metadata in device buffers (:class:`vgate.runtime.step_meta.StepView`),
as for the transformer families, so the same code is captured into a hipGraph per bucket.

Layer arrangements (``ARRANGEMENTS``, chosen by ``HybridArch.arrangement``):
  gated_parallel  h  = x / sqrt(mean(x^2) + eps) * g          one scalar weight per norm
                  P  = h @ [mixer inputs; rg1; rg2]^T         ONE fused input projection per layer
                  x += mixer(h) * sigmoid(P_rg1 + b1) + ff(h) * sigmoid(P_rg2 + b2)
  post_norm       x += rmsnorm(mixer(x)) * w1;  x += rmsnorm(ff(x)) * w2
                  (the sublayers read the stream itself, rounded to the activation dtype; their
                  outputs are normed in fp32 before they are added)
  hyper_pre_norm  ``HybridArch.streams`` fp32 copies x_1 .. x_S of the stream (all equal to the embedding
                  output at the start); per sublayer q with a tanh norm (no statistics):
                  u = sum_s in_q[s] x_s;  y = sublayer(tanh(alpha u) * w + b);
                  x_t <- sum_s mix_q[s, t] x_s + out_q[t] y   (all copies at once); the model's result
                  is the sum of the copies
  pre_norm        x += m * mixer(rmsnorm(x) * w1);  x += m * ff(rmsnorm(x) * w2)   (m = ``residual_mult``; a
                  sublayer's add and the next sublayer's norm are one kernel)
``HybridArch.loop`` = (start, stop, times): the layers start .. stop - 1 run ``times`` times in a row with the same
weights, every pass with caches and states of its own; right before the first layer of each pass the stream
becomes W_in [x; x0] (``loop.in``, x0 the embedding output).
With ``HybridArch.depth_average`` the stream a layer hands on is a learned combination of the
embedding output X_0 and every layer result X_1 .. X_(i+1): sum_j c_i[j] X_j (tensor ``l<i>.dwa``).
A layer may run with another layer's weights (``weights_of``) while keeping its own cache or state.
Activation dtype bf16 (MFMA GEMMs, fp32 accumulation) or fp32 (true fp32 FMA everywhere); the residual
stream, norms, scores, routers and recurrent state are fp32 in both.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch

from vgate.models.config import HybridArch
from vgate.models.mixers import FEED_FORWARDS, MIXERS, Proj, _f32, _pad8
from vgate.ops import seq
from vgate.parallel.comm import TPGroup


def _fuse_inputs(mixer, extra: list, width: int, device, f32: bool):
    """Stack every matrix that multiplies the layer's input into ONE GEMM (segments padded to 8 rows,
    the total to 64 columns). Returns (Proj, {name: (first column, columns)})."""
    rows = list(mixer.in_rows) + extra
    if not rows:   # a mixer whose projections all read inputs of their own
        del mixer.in_rows
        return None, {}
    biases = dict(getattr(mixer, "in_bias", {}))
    col, parts, bparts, off = {}, [], [], 0
    for name, w in rows:
        col[name] = (off, w.shape[0])
        b = biases.get(name)
        b = torch.zeros(w.shape[0], dtype=w.dtype) if b is None else b
        w = _pad8(w)
        parts.append(w)
        bparts.append(torch.cat([b, torch.zeros(w.shape[0] - b.shape[0], dtype=b.dtype)]))
        off += w.shape[0]
    if off % 64:  # whole 64-column tiles: the widest alignment any of the GEMMs asks for
        parts.append(torch.zeros(64 - off % 64, width, dtype=parts[0].dtype))
        bparts.append(torch.zeros(64 - off % 64, dtype=bparts[0].dtype))
    del mixer.in_rows
    return Proj(torch.cat(parts), device, f32, bias=torch.cat(bparts) if biases else None), col


class GatedParallelLayer:
    """The tensors of one weight-owning layer of the ``gated_parallel`` arrangement in kernel-ready form."""

    def __init__(self, spec, width: int, eps: float, t: dict, device, f32: bool):
        mix = {k[4:]: v for k, v in t.items() if k.startswith("mix.")}
        self.eps = eps
        self.mixer = MIXERS[spec.kind](spec.mixer, width, eps, mix, device, f32)
        if spec.kind == "parallel":
            raise ValueError("the gated_parallel arrangement takes single mixers")
        self.ff = None
        if spec.mlp:
            mlp = {k[4:]: v for k, v in t.items() if k.startswith("mlp.")}
            self.ff = FEED_FORWARDS[spec.mlp["kind"]](spec.mlp, width, mlp, device, f32)
        self.norm1 = _f32(t["norm1"].reshape(1), device)
        extra = [("rg1", t["rg1"])]
        self.rg1_b = _f32(t["rg1.b"], device)
        self.rg2_b = None
        if self.ff is not None:
            extra.append(("rg2", t["rg2"]))
            self.rg2_b = _f32(t["rg2.b"], device)
        self.proj, self.col = _fuse_inputs(self.mixer, extra, width, device, f32)

    @staticmethod
    def shapes(spec, width: int) -> dict:
        out = {"norm1": ()}
        out.update({"mix." + k: v for k, v in MIXERS[spec.kind].shapes(spec.mixer, width).items()})
        out.update({"rg1": (width, width), "rg1.b": (width,)})
        if spec.mlp:
            out.update({"mlp." + k: v for k, v in FEED_FORWARDS[spec.mlp["kind"]].shapes(spec.mlp, width).items()})
            out.update({"rg2": (width, width), "rg2.b": (width,)})
        return out

    def cols(self, P: torch.Tensor, name: str) -> torch.Tensor:
        a, n = self.col[name]
        return P[:, a: a + n]

    def nbytes(self) -> int:
        return self.proj.nbytes() + self.mixer.nbytes() + (self.ff.nbytes() if self.ff else 0)

    def run(self, st, sv, cache) -> None:
        x, h = st.x, st.h
        seq.norm_rows(x, self.norm1, self.eps, h, scalar=True)
        P = self.proj(h)
        y1 = self.mixer.forward(h, P, self.cols, sv, cache)
        y2 = self.ff.forward(h) if self.ff is not None else None
        seq.gated_residual(x, y1, self.cols(P, "rg1"), self.rg1_b, y2, self.cols(P, "rg2") if y2 is not None else None,
                           self.rg2_b)


class PostNormLayer:
    """``post_norm`` arrangement: the mixer and the feed-forward read the stream itself; each output is
    RMS-normed (vector weight, fp32) and then added. The residual kernel also hands on the activation-
    dtype copy the next GEMM reads and, for the layer's last sublayer, the depth average."""

    def __init__(self, spec, width: int, eps: float, t: dict, device, f32: bool):
        mix = {k[4:]: v for k, v in t.items() if k.startswith("mix.")}
        self.eps = eps
        self.mixer = MIXERS[spec.kind](spec.mixer, width, eps, mix, device, f32)
        self.norm1 = _f32(t["norm1"], device)
        self.ff = self.norm2 = None
        if spec.mlp:
            mlp = {k[4:]: v for k, v in t.items() if k.startswith("mlp.")}
            self.ff = FEED_FORWARDS[spec.mlp["kind"]](spec.mlp, width, mlp, device, f32)
            self.norm2 = _f32(t["norm2"], device)
        self.dwa = _f32(t["dwa"], device) if "dwa" in t else None
        self.proj, self.col = _fuse_inputs(self.mixer, [], width, device, f32)

    @staticmethod
    def shapes(spec, width: int) -> dict:
        out = {"norm1": (width,)}
        out.update({"mix." + k: v for k, v in MIXERS[spec.kind].shapes(spec.mixer, width).items()})
        if spec.mlp:
            out.update({"mlp." + k: v for k, v in FEED_FORWARDS[spec.mlp["kind"]].shapes(spec.mlp, width).items()})
            out["norm2"] = (width,)
        return out

    def cols(self, P: torch.Tensor, name: str) -> torch.Tensor:
        a, n = self.col[name]
        return P[:, a: a + n]

    def nbytes(self) -> int:
        return self.proj.nbytes() + self.mixer.nbytes() + (self.ff.nbytes() if self.ff else 0)

    def run(self, st, sv, cache) -> None:
        """st.x: the stream entering the layer (fp32), st.h its activation-dtype copy; the layer's result
        goes to st.result (plane i + 1 of the history when the model averages over depth) and what the
        next layer reads replaces st.x / st.h."""
        P = self.proj(st.h)
        y = self.mixer.forward(st.h, P, self.cols, sv, cache)
        y1, s1, y2, s2 = y if isinstance(y, tuple) else (y, 1.0, None, 1.0)
        last = self.ff is None
        seq.post_norm_add(st.x, y1, self.norm1, self.eps, st.result, s1=s1, y2=y2, s2=s2, **st.hand_on(last))
        if not last:
            yf = self.ff.forward(st.result if st.f32 else st.h, out_f32=True)
            seq.post_norm_add(st.result, yf, self.norm2, self.eps, st.result, **st.hand_on(True))


class _TanhNorm:
    """tanh(alpha x) * w + b: the tensors ``<name>`` [W], ``<name>.b`` [W], ``<name>.alpha`` []."""

    def __init__(self, t: dict, name: str, device):
        self.alpha = _f32(t[name + ".alpha"].reshape(1), device)
        self.w, self.b = _f32(t[name], device), _f32(t[name + ".b"], device)

    @staticmethod
    def shapes(name: str, width: int) -> dict:
        return {name: (width,), name + ".b": (width,), name + ".alpha": ()}


class HyperPreNormLayer:
    """``hyper_pre_norm`` arrangement: every sublayer reads a learned combination of the stream's copies
    through a tanh norm and writes back to all of them (tensors ``hc<q>.in`` [S], ``hc<q>.out`` [S],
    ``hc<q>.mix`` [S from, S to]). A sublayer's write and the next sublayer's read (also the next layer's,
    or the final sum over the copies) are one kernel."""

    def __init__(self, spec, width: int, eps: float, t: dict, device, f32: bool):
        mix = {k[4:]: v for k, v in t.items() if k.startswith("mix.")}
        self.eps = eps
        if spec.kind == "parallel":
            raise ValueError("the hyper_pre_norm arrangement takes single mixers")
        self.mixer = MIXERS[spec.kind](spec.mixer, width, eps, mix, device, f32)
        self.norm1 = _TanhNorm(t, "norm1", device)
        self.hc = [tuple(_f32(t[f"hc1.{n}"], device) for n in ("in", "out", "mix"))]
        self.ff = self.norm2 = None
        if spec.mlp:
            mlp = {k[4:]: v for k, v in t.items() if k.startswith("mlp.")}
            self.ff = FEED_FORWARDS[spec.mlp["kind"]](spec.mlp, width, mlp, device, f32)
            self.norm2 = _TanhNorm(t, "norm2", device)
            self.hc.append(tuple(_f32(t[f"hc2.{n}"], device) for n in ("in", "out", "mix")))
        S = self.hc[0][0].numel()
        if S > seq.MAX_STREAMS or any(c[2].shape != (S, S) or c[1].numel() != S for c in self.hc):
            raise ValueError(f"hyper_pre_norm: 1 .. {seq.MAX_STREAMS} copies, mix [copies, copies]")
        self.proj, self.col = _fuse_inputs(self.mixer, [], width, device, f32)

    @staticmethod
    def shapes(spec, width: int, streams: int = 1) -> dict:
        hc = lambda q: {f"hc{q}.in": (streams,), f"hc{q}.out": (streams,), f"hc{q}.mix": (streams, streams)}  # noqa: E731
        out = dict(_TanhNorm.shapes("norm1", width))
        out.update({"mix." + k: v for k, v in MIXERS[spec.kind].shapes(spec.mixer, width).items()})
        out.update(hc(1))
        if spec.mlp:
            out.update({"mlp." + k: v for k, v in FEED_FORWARDS[spec.mlp["kind"]].shapes(spec.mlp, width).items()})
            out.update(_TanhNorm.shapes("norm2", width))
            out.update(hc(2))
        return out

    def cols(self, P: torch.Tensor, name: str) -> torch.Tensor:
        a, n = self.col[name]
        return P[:, a: a + n]

    def nbytes(self) -> int:
        return self.proj.nbytes() + self.mixer.nbytes() + (self.ff.nbytes() if self.ff else 0)

    def reader(self) -> tuple:
        """What the kernel before this layer needs to prepare its first sublayer's input."""
        return self.hc[0][0], self.norm1

    def run(self, st, sv, cache) -> None:
        """st.xs [S, T, W]: the copies; st.h: the first sublayer's normed input, made by the write before
        (the embedding's, or the previous layer's last). st.next_reader: the next layer's (None: the last)."""
        P = self.proj(st.h)
        y = self.mixer.forward(st.h, P, self.cols, sv, cache)
        _, out_w, mix = self.hc[0]
        if self.ff is not None:
            st.write(y, mix, out_w, (self.hc[1][0], self.norm2))
            y = self.ff.forward(st.h, out_f32=True)
            _, out_w, mix = self.hc[1]
        st.write(y, mix, out_w, st.next_reader)


class PreNormLayer:
    """``pre_norm`` arrangement: x += mult * mixer(rmsnorm(x) * norm1), then x += mult * ff(rmsnorm(x) * norm2)
    (vector weights, fp32 statistics). The residual kernel of a sublayer also makes the normed input of the
    sublayer that follows (the feed-forward's, or the next layer's first when the model says which that is)."""

    def __init__(self, spec, width: int, eps: float, t: dict, device, f32: bool, mult: float = 1.0):
        mix = {k[4:]: v for k, v in t.items() if k.startswith("mix.")}
        self.eps, self.mult = eps, float(mult)
        if spec.kind == "parallel":
            raise ValueError("the pre_norm arrangement takes single mixers")
        self.mixer = MIXERS[spec.kind](spec.mixer, width, eps, mix, device, f32)
        self.norm1 = _f32(t["norm1"], device)
        self.ff = self.norm2 = None
        if spec.mlp:
            mlp = {k[4:]: v for k, v in t.items() if k.startswith("mlp.")}
            self.ff = FEED_FORWARDS[spec.mlp["kind"]](spec.mlp, width, mlp, device, f32)
            self.norm2 = _f32(t["norm2"], device)
        self.proj, self.col = _fuse_inputs(self.mixer, [], width, device, f32)

    @staticmethod
    def shapes(spec, width: int) -> dict:
        out = {"norm1": (width,)}
        out.update({"mix." + k: v for k, v in MIXERS[spec.kind].shapes(spec.mixer, width).items()})
        if spec.mlp:
            out.update({"mlp." + k: v for k, v in FEED_FORWARDS[spec.mlp["kind"]].shapes(spec.mlp, width).items()})
            out["norm2"] = (width,)
        return out

    def cols(self, P: torch.Tensor, name: str) -> torch.Tensor:
        a, n = self.col[name]
        return P[:, a: a + n]

    def nbytes(self) -> int:
        return (self.proj.nbytes() if self.proj else 0) + self.mixer.nbytes() + (self.ff.nbytes() if self.ff else 0)

    def run(self, st, sv, cache) -> None:
        """st.x: the fp32 stream; st.h: the normed input in the activation dtype (``st.h_ready``: the kernel before
        has made this layer's already); st.next_norm: the norm weight of the layer that follows, or None."""
        if not st.h_ready:
            seq.norm_rows(st.x, self.norm1, self.eps, st.h)
        P = self.proj(st.h) if self.proj is not None else None
        y = self.mixer.forward(st.h, P, self.cols, sv, cache)
        if self.ff is not None:
            seq.residual_norm(st.x, y, self.mult, self.norm2, self.eps, st.h)
            y = self.ff.forward(st.h, out_f32=True)
        seq.residual_norm(st.x, y, self.mult, st.next_norm, self.eps, st.h if st.next_norm is not None else None)
        st.h_ready = st.next_norm is not None


class _PreStream:
    """The stream of one ``pre_norm`` step: ``x`` fp32 [T, W], ``h`` the next sublayer's normed input."""

    def __init__(self, T: int, W: int, act_dtype, device):
        self.x = torch.empty(T, W, dtype=torch.float32, device=device)
        self.h = torch.empty(T, W, dtype=act_dtype, device=device)
        self.h_ready, self.next_norm = False, None


ARRANGEMENTS = {"gated_parallel": GatedParallelLayer, "post_norm": PostNormLayer, "hyper_pre_norm": HyperPreNormLayer,
                "pre_norm": PreNormLayer}


class _HyperStream:
    """The stream's copies of one step: ``xs`` fp32 [S, T, W], ``h`` the next sublayer's normed input in the
    activation dtype, ``x`` (after the last layer's write) the sum of the copies."""

    def __init__(self, S: int, T: int, W: int, act_dtype, device, keep_sums: bool):
        self.xs = torch.empty(S, T, W, dtype=torch.float32, device=device)
        self.h = torch.empty(T, W, dtype=act_dtype, device=device)
        self.x = torch.empty(T, W, dtype=torch.float32, device=device)
        self.next_reader, self.keep_sums = None, keep_sums

    def write(self, y, mix, out_w, reader) -> None:
        rd = {} if reader is None else dict(read_w=reader[0], alpha=reader[1].alpha, w=reader[1].w, b=reader[1].b, h_out=self.h)
        last = reader is None or (self.keep_sums and reader is self.next_reader)
        seq.hyper_mix(self.xs, y, mix, out_w, sum_out=self.x if last else None, **rd)


class _Stream:
    """The residual stream of one step: ``x`` fp32 [T, W] and ``h``, its copy in the activation dtype
    (``x`` itself in an fp32 model). With depth averaging ``hist`` [layers + 1, T, W] keeps the
    embedding output and every layer's result, and ``x`` is the average the next layer reads."""

    def __init__(self, T: int, W: int, layers: int, act_dtype, device, depth_average: bool, normed_input: bool):
        # an fp32 model whose sublayers read the stream itself needs no copy: h is x
        self.f32 = act_dtype == torch.float32 and not normed_input
        self.hist = torch.empty(layers + 1, T, W, dtype=torch.float32, device=device) if depth_average else None
        self.x = self.hist[0] if depth_average else torch.empty(T, W, dtype=torch.float32, device=device)
        self.h = self.x if self.f32 else torch.empty(T, W, dtype=act_dtype, device=device)
        self.mix = torch.empty(T, W, dtype=torch.float32, device=device) if depth_average else None
        self.result, self.layer, self.coef = self.x, 0, None

    def begin(self, i: int, coef) -> None:
        self.layer, self.coef = i, coef
        self.result = self.hist[i + 1] if self.hist is not None else self.x

    def hand_on(self, last: bool) -> dict:
        """Extra outputs of a residual kernel: the activation-dtype copy of what the next GEMM reads and,
        after the layer's last sublayer, the depth average (which then is what the copy is made of)."""
        kw = {}
        if last and self.hist is not None:
            kw.update(hist=self.hist, planes=self.layer + 2, coef=self.coef, mix=self.mix)
        if not self.f32:
            kw["act_out"] = self.h
        return kw

    def end(self) -> None:
        if self.hist is not None:
            self.x = self.mix
            if self.f32:
                self.h = self.x
        # (without depth averaging the result was written over x in place)


class HybridModel:
    stateful = True  # recurrent state: no prefix reuse, no recompute from a cached prefix

    def __init__(self, arch: HybridArch, device, tp: TPGroup | None = None, quantization: str | None = None,
                 seed: int = 0, weights_path: str | None = None, max_model_len: int = 4096,
                 dtype: str = "bfloat16"):
        self.arch = arch
        self.device = torch.device(device)
        self.tp = tp or TPGroup()
        if self.tp.size > 1:
            raise ValueError("layered hybrid models run on one GPU per replica (tensor_parallel_size 1)")
        if (quantization or "none").lower() not in ("none", ""):
            raise ValueError(f"layered hybrid models have no quantized path (quantization={quantization!r})")
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype {dtype!r}: bfloat16 or float32")
        self.f32 = dtype == "float32"
        self.act_dtype = torch.float32 if self.f32 else torch.bfloat16
        self.max_model_len = max_model_len
        W = arch.hidden_size
        tensors = load_tensors(arch, weights_path) if weights_path else random_tensors(arch, seed)
        self.embed = tensors["embed"].to(self.device, self.act_dtype).contiguous()
        layer_cls = ARRANGEMENTS[arch.arrangement]
        extra = {"mult": arch.residual_mult} if arch.arrangement == "pre_norm" else {}
        owned: dict = {}
        self.layers: list = []        # one entry per layer RUN (a looped layer once per pass): caches are per run
        self.pass_start: list = []    # whether a pass of the loop starts at that run
        for i, first in arch.run_order():
            spec = arch.layers[i]
            j = arch.owner(i)
            if j not in owned:
                pre = f"l{j}."
                t = {k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}
                owned[j] = layer_cls(arch.layers[j], W, arch.rms_eps, t, self.device, self.f32, **extra)
            if MIXERS[spec.kind] is not type(owned[j].mixer):
                raise ValueError(f"layer {i} shares weights with layer {j} of another mixer type")
            self.layers.append(owned[j])
            self.pass_start.append(first)
        self._owned = owned
        self.loop_in = Proj(tensors["loop.in"], self.device, self.f32) if arch.loop is not None else None
        # depth-average coefficients belong to the position in the stack, not to the (possibly shared) weights
        self.depth_coef = [_f32(tensors[f"l{i}.dwa"], self.device) for i in range(arch.num_layers)] \
            if arch.depth_average else None
        self.scalar_norm = arch.arrangement == "gated_parallel"   # one number per norm, or a weight vector
        self.hyper = arch.arrangement == "hyper_pre_norm"
        self.final_norm = _TanhNorm(tensors, "final.norm", self.device) if self.hyper else \
            _f32(tensors["final.norm"].reshape(-1), self.device)
        if arch.logit_scale != 1.0:   # logits = head (norm(x) w) s = head (norm(x) (w s)): one fp32 product, made here
            if self.hyper:
                raise ValueError("a logit scale needs an RMS final norm")
            self.final_norm = self.final_norm * arch.logit_scale
        self.head = Proj(tensors["embed" if arch.tie_embeddings else "head"], self.device, self.f32)
        self.capture_layers: list | None = None  # set to [] to record the residual stream after every layer
        self.last_resid = None

    # ------------------------------------------------------------------ sizes
    def weight_bytes(self) -> int:
        return (self.embed.numel() * self.embed.element_size() + self.head.nbytes()
                + sum(L.nbytes() for L in self._owned.values()))

    def cache_bytes_per_block(self, block_size: int) -> int:
        """Bytes one cache page costs over all layers with a paged cache."""
        return max(sum(L.mixer.page_bytes(block_size) for L in self.layers), 1)

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int) -> list:
        """Per layer what its mixer keeps between steps: a paged cache, a state [slots, ...], or a tuple
        of these (zeroed: stale rows are always finite)."""
        return [L.mixer.allocate(num_blocks, block_size, num_slots, self.device) for L in self.layers]

    # ---------------------------------------------------------------- forward
    def forward(self, sv, caches, part_size: int = 0, return_hidden: bool = False) -> torch.Tensor:
        """One step. Returns fp32 logits [S, vocab] of the sample rows, or with ``return_hidden`` the
        fp32 residual stream [T, width] after the last layer."""
        if self.hyper or self.arch.arrangement == "pre_norm":
            x = self._forward_hyper(sv, caches) if self.hyper else self._forward_pre(sv, caches)
            return x if return_hidden else self._padded_logits(x, sv)
        T = sv.T
        W = self.arch.hidden_size
        dev, eps = self.device, self.arch.rms_eps
        st = _Stream(T, W, len(self.layers), self.act_dtype, dev, self.arch.depth_average,
                     normed_input=self.arch.arrangement != "post_norm")
        seq.embed_rows(sv.ids, self.embed, st.x, prev=sv.prev_tokens)
        if self.arch.arrangement == "post_norm" and not self.f32:
            seq.cast_rows(st.x, st.h)   # (the gated_parallel arrangement makes h with its norm)
        for li, L in enumerate(self.layers):
            st.begin(li, self.depth_coef[li] if self.depth_coef else None)
            L.run(st, sv, caches[li])
            st.end()
            if self.capture_layers is not None:
                self.capture_layers.append(st.x.clone())
        x = st.x
        self.last_resid = x
        if return_hidden:
            return x
        return self._padded_logits(x, sv)

    def _forward_hyper(self, sv, caches) -> torch.Tensor:
        """The layer loop over several copies of the stream; returns their sum, fp32 [T, width]."""
        S, T, W = self.arch.streams, sv.T, self.arch.hidden_size
        st = _HyperStream(S, T, W, self.act_dtype, self.device, keep_sums=self.capture_layers is not None)
        seq.embed_rows(sv.ids, self.embed, st.xs[0], prev=sv.prev_tokens)
        for s in range(1, S):
            st.xs[s].copy_(st.xs[0])
        first = self.layers[0].reader()
        st.next_reader = first
        st.write(None, None, None, first)   # the first sublayer's input (nothing to add yet)
        for li, L in enumerate(self.layers):
            st.next_reader = self.layers[li + 1].reader() if li + 1 < len(self.layers) else None
            L.run(st, sv, caches[li])
            if self.capture_layers is not None:
                self.capture_layers.append(st.x.clone())
        self.last_resid = st.x
        return st.x

    def _forward_pre(self, sv, caches) -> torch.Tensor:
        """The layer loop of the ``pre_norm`` arrangement, with the looped stretch; returns the fp32 stream."""
        T, W = sv.T, self.arch.hidden_size
        st = _PreStream(T, W, self.act_dtype, self.device)
        seq.embed_rows(sv.ids, self.embed, st.x, prev=sv.prev_tokens)
        x0 = pair = None
        if self.loop_in is not None:
            x0 = st.x.clone()
            pair = torch.empty(T, 2 * W, dtype=self.act_dtype, device=self.device)
        n = len(self.layers)
        for ri, L in enumerate(self.layers):
            if self.pass_start[ri]:   # x <- W_in [x; x0]
                seq.pair_rows(st.x, x0, pair)
                self.loop_in(pair, out_f32=True, out=st.x)
                st.h_ready = False
            nxt = self.layers[ri + 1] if ri + 1 < n and not self.pass_start[ri + 1] else None
            st.next_norm = nxt.norm1 if nxt is not None else None
            L.run(st, sv, caches[ri])
            if self.capture_layers is not None:
                self.capture_layers.append(st.x.clone())
        self.last_resid = st.x
        return st.x

    def _padded_logits(self, x: torch.Tensor, sv) -> torch.Tensor:
        dev = x.device
        V = self.arch.vocab_size
        if V % 4 == 0:
            return self.logits_of(x, sv.sample_idx)
        # the sampler reads rows of whole 16-B pieces: pad the row with -inf columns (never sampled)
        buf = torch.full((sv.sample_idx.numel(), (V + 3) // 4 * 4), float("-inf"), dtype=torch.float32, device=dev)
        self.logits_of(x, sv.sample_idx, out=buf[:, :V])
        return buf

    def logits_of(self, x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """fp32 logits [len(rows), vocab] of rows of the residual stream (final norm + head)."""
        hn = torch.empty(rows.numel(), x.shape[1], dtype=self.act_dtype, device=x.device)
        if self.hyper:
            n = self.final_norm
            seq.tanh_norm_rows(x, n.alpha, n.w, n.b, hn, rows=rows)
        else:
            seq.norm_rows(x, self.final_norm, self.arch.rms_eps, hn, rows=rows, scalar=self.scalar_norm)
        return self.head(hn, out_f32=True, out=out)[:, : self.arch.vocab_size]


# ------------------------------------------------------------------------------------------ weights
def tensor_shapes(arch: HybridArch, nominal: int | None = 16) -> dict:
    """name -> shape of every tensor of a checkpoint of ``arch`` (weight-owning layers only). A size
    that only a checkpoint's tensors give (a low-rank gate's width) is ``nominal``; None leaves it open."""
    W = arch.hidden_size
    vector = arch.arrangement != "gated_parallel"
    out = {"embed": (arch.vocab_size, W), "final.norm": (W,) if vector else ()}
    if not arch.tie_embeddings:
        out["head"] = (arch.vocab_size, W)
    if arch.loop is not None:
        out["loop.in"] = (W, 2 * W)
    extra = {}
    if arch.arrangement == "hyper_pre_norm":
        out.update(_TanhNorm.shapes("final.norm", W))
        extra = {"streams": arch.streams}
    for i in sorted({arch.owner(i) for i in range(arch.num_layers)}):
        out.update({f"l{i}.{k}": v for k, v in ARRANGEMENTS[arch.arrangement].shapes(arch.layers[i], W, **extra).items()})
    if arch.depth_average:
        out.update({f"l{i}.dwa": (i + 2,) for i in range(arch.num_layers)})
    return {k: tuple(nominal if d is None else d for d in v) for k, v in out.items()}


def load_tensors(arch: HybridArch, path: str) -> dict:
    """Read ``model.safetensors`` (bf16 tensors, row-major [out, in]) of a layered hybrid checkpoint
    and check every tensor the architecture needs against its expected shape. Sizes the config does
    not carry (the decay low-rank width) come from the tensors."""
    from safetensors import safe_open
    root = Path(path)
    files = sorted(root.glob("*.safetensors")) if root.is_dir() else [root]
    if not files:
        raise FileNotFoundError(f"no *.safetensors under {root}")
    t = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as h:
            for k in h.keys():
                t[k] = h.get_tensor(k)
    for name, shape in tensor_shapes(arch, nominal=None).items():
        if name not in t:
            raise KeyError(f"checkpoint lacks tensor {name}")
        got = tuple(t[name].shape)
        if None in shape:   # a size only the tensors give (the mixer checks that its tensors agree on it)
            ok = len(got) == len(shape) and all(w is None or g == w for g, w in zip(got, shape))
        else:
            ok = got == tuple(shape) or (math.prod(got) == 1 and math.prod(shape) == 1)
        if not ok:
            raise ValueError(f"tensor {name}: shape {got}, expected {tuple(shape)}")
    return t


def random_tensors(arch: HybridArch, seed: int = 0) -> dict:
    """Seeded random bf16 weights (benchmarks / tests): matrices ~ N(0, 1 / fan_in), norm weights near 1,
    biases and corrections small, so activations stay O(1) through any depth."""
    g = torch.Generator().manual_seed(seed * 1000003 + 17)
    out = {}
    for name, shape in tensor_shapes(arch).items():
        leaf = name.split(".")[-1] if not name.endswith(".b") else "b"
        hyper = ".hc" in name
        if leaf == "dwa":  # close to "hand on the newest result"
            w = 0.1 * torch.randn(shape, generator=g) / shape[0]
            w[-1] += 1.0
        elif hyper and leaf == "mix":    # close to "every copy keeps itself"
            w = torch.eye(shape[0]) + 0.2 * torch.randn(shape, generator=g)
        elif hyper and leaf == "in":
            w = (1.0 + 0.3 * torch.randn(shape, generator=g)) / shape[0]
        elif hyper and leaf == "out":
            w = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif ".mu." in name:             # a blend weight between the token and the one before
            w = torch.rand(shape, generator=g)
        elif name == "loop.in":          # close to "keep the stream": [I, 0] plus noise
            w = torch.cat([torch.eye(shape[0]), torch.zeros(shape[0], shape[0])], 1) + torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif leaf in ("alpha", "temp"):  # positive, near 1
            w = 0.8 + 0.2 * torch.rand(shape, generator=g)
        elif leaf in ("r1", "r2"):       # positive: ln(1 + r2 * distance) must exist
            w = 0.05 + 0.5 * torch.rand(shape, generator=g)
        elif len(shape) == 2:
            std = 0.5 if name == "embed" else 1.0 / math.sqrt(shape[1])
            w = torch.randn(shape, generator=g) * std
        elif leaf in ("norm", "norm1", "norm2") or name == "final.norm":
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        else:
            w = 0.3 * torch.randn(shape, generator=g)
        out[name] = w.to(torch.bfloat16)
    return out


def save_checkpoint(arch: HybridArch, tensors: dict, path: str, config: dict) -> None:
    """Write ``config.json`` + ``model.safetensors`` of a layered hybrid model."""
    from safetensors.torch import save_file
    Path(path).mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(Path(path) / "model.safetensors"))
    (Path(path) / "config.json").write_text(json.dumps(config, indent=1))
