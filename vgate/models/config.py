"""Model architecture descriptions (Qwen2 / Llama family decoder-only transformers).

Dimensions are the public HF ``config.json`` values of each model.
A model id resolves to an :class:`ModelArch` either by a local directory holding a
``config.json`` (real checkpoint) or by a built-in preset matched on the id's
name (random-init weights, used for benchmarks: there are no checkpoints here).
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import asdict, dataclass, field, replace
from pathlib import Path


@dataclass(frozen=True)
class ModelArch:
    name: str
    family: str  # "qwen2" | "llama"
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_eps: float = 1e-6
    rope_theta: float = 10000.0
    rope_scaling: dict | None = field(default=None, hash=False, compare=False)
    qkv_bias: bool = False
    tie_embeddings: bool = False
    max_position: int = 32768
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        H, I, V, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_layers
        per_layer = H * (self.q_size + 2 * self.kv_size) + self.q_size * H + 3 * H * I + 2 * H
        if self.qkv_bias:
            per_layer += self.q_size + 2 * self.kv_size
        emb = V * H * (1 if self.tie_embeddings else 2)
        return L * per_layer + emb + H

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.num_layers * self.kv_size * dtype_bytes

    def to_dict(self) -> dict:
        return asdict(self)


PRESETS: dict[str, ModelArch] = {
    "qwen2.5-0.5b": ModelArch("qwen2.5-0.5b", "qwen2", 896, 24, 14, 2, 64, 4864, 151936, 1e-6, 1e6,
                              qkv_bias=True, tie_embeddings=True, bos_token_id=151643,
                              eos_token_ids=(151645, 151643)),
    "qwen2.5-1.5b": ModelArch("qwen2.5-1.5b", "qwen2", 1536, 28, 12, 2, 128, 8960, 151936, 1e-6, 1e6,
                              qkv_bias=True, tie_embeddings=True, bos_token_id=151643,
                              eos_token_ids=(151645, 151643)),
    "qwen2.5-7b": ModelArch("qwen2.5-7b", "qwen2", 3584, 28, 28, 4, 128, 18944, 152064, 1e-6, 1e6,
                            qkv_bias=True, tie_embeddings=False, bos_token_id=151643,
                            eos_token_ids=(151645, 151643)),
    "llama-3-8b": ModelArch("llama-3-8b", "llama", 4096, 32, 32, 8, 128, 14336, 128256, 1e-5, 5e5,
                            max_position=8192, bos_token_id=128000, eos_token_ids=(128001, 128009)),
    "llama-3.1-8b": ModelArch("llama-3.1-8b", "llama", 4096, 32, 32, 8, 128, 14336, 128256, 1e-5, 5e5,
                              rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                            "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
                              max_position=131072, bos_token_id=128000, eos_token_ids=(128001, 128009)),
    "llama-3-70b": ModelArch("llama-3-70b", "llama", 8192, 80, 64, 8, 128, 28672, 128256, 1e-5, 5e5,
                             max_position=8192, bos_token_id=128000, eos_token_ids=(128001, 128009)),
    # small configs for tests / CPU smoke (head_dim must stay 128 for the GPU kernels)
    "tiny": ModelArch("tiny", "qwen2", 256, 2, 4, 2, 128, 512, 512, 1e-6, 1e4, qkv_bias=True,
                      tie_embeddings=True, max_position=4096, bos_token_id=1, eos_token_ids=(2,)),
    "tiny-llama": ModelArch("tiny-llama", "llama", 256, 2, 4, 1, 128, 384, 1024, 1e-5, 5e5,
                            max_position=4096, bos_token_id=1, eos_token_ids=(2,)),
    # TP tests up to 8 ranks: 8 query heads, 2 KV heads (replicated at TP 4 / 8), a vocabulary
    # that is not a multiple of 16 * 8 (padded vocab shards)
    "tiny-tp8": ModelArch("tiny-tp8", "qwen2", 256, 2, 8, 2, 128, 1024, 500, 1e-6, 1e4, qkv_bias=True,
                          tie_embeddings=True, max_position=4096, bos_token_id=1, eos_token_ids=(2,)),
}

_ALIASES = [
    ("qwen2.5-0.5b", "qwen2.5-0.5b"),
    ("qwen2.5-1.5b", "qwen2.5-1.5b"),
    ("qwen2.5-7b", "qwen2.5-7b"),
    ("llama-3.1-8b", "llama-3.1-8b"),
    ("llama-3-70b", "llama-3-70b"),
    ("meta-llama-3-70b", "llama-3-70b"),
    ("llama-3-8b", "llama-3-8b"),
    ("meta-llama-3-8b", "llama-3-8b"),
    ("tiny-llama", "tiny-llama"),
    ("tiny-tp8", "tiny-tp8"),
    ("tiny", "tiny"),
]


def _from_hf_config(cfg: dict, name: str) -> ModelArch:
    mt = cfg.get("model_type", "llama")
    family = "qwen2" if mt.startswith("qwen2") else "llama"
    H = cfg["hidden_size"]
    nh = cfg["num_attention_heads"]
    eos = cfg.get("eos_token_id", 2)
    eos = tuple(eos) if isinstance(eos, list) else (eos,)
    return ModelArch(
        name=name, family=family, hidden_size=H, num_layers=cfg["num_hidden_layers"], num_heads=nh,
        num_kv_heads=cfg.get("num_key_value_heads", nh), head_dim=cfg.get("head_dim", H // nh),
        intermediate_size=cfg["intermediate_size"], vocab_size=cfg["vocab_size"],
        rms_eps=cfg.get("rms_norm_eps", 1e-6), rope_theta=cfg.get("rope_theta", 10000.0),
        rope_scaling=cfg.get("rope_scaling"), qkv_bias=(family == "qwen2") or cfg.get("attention_bias", False),
        tie_embeddings=cfg.get("tie_word_embeddings", False),
        max_position=cfg.get("max_position_embeddings", 32768),
        bos_token_id=cfg.get("bos_token_id", 1) or 1, eos_token_ids=eos)


@dataclass(frozen=True)
class LayerSpec:
    """One layer of a layered hybrid model: which mixer it has (a key of
    ``vgate.models.mixers.MIXERS``), the mixer's sizes and constants, its feed-forward (``None``:
    the layer has none) and, for a layer without tensors of its own, the layer whose weights it
    runs with (its cache or state stays its own)."""
    kind: str
    mixer: dict = field(hash=False, compare=False)
    mlp: dict | None = field(default=None, hash=False, compare=False)
    weights_of: int | None = None


@dataclass(frozen=True)
class HybridArch:
    """A decoder made of a list of :class:`LayerSpec` over an fp32 residual stream."""
    name: str
    family: str
    hidden_size: int
    vocab_size: int
    layers: tuple
    rms_eps: float = 1e-6
    max_position: int = 1 << 20
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)
    # how a layer combines its sublayers (a key of ``vgate.models.hybrid.ARRANGEMENTS``) and whether
    # the stream that enters the next layer is a learned average of all earlier layers' results
    arrangement: str = "gated_parallel"
    depth_average: bool = False
    # copies of the residual stream a layer reads and writes through learned weights (1: one plain stream);
    # the ``hyper_pre_norm`` arrangement uses them
    streams: int = 1
    # ``pre_norm`` arrangement: every sublayer's result is multiplied by this before it is added
    residual_mult: float = 1.0
    # (start, stop, times): layers start .. stop - 1 run ``times`` times in a row with the same weights, every
    # pass with caches and states of its own; right before the first layer of each pass the stream is replaced by
    # W_in [x; x0] (tensor ``loop.in`` [width, 2 width], x0 the embedding output)
    loop: tuple | None = None
    # the logits are multiplied by this; with ``tie_embeddings`` the embedding table is the output matrix
    logit_scale: float = 1.0
    tie_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def run_order(self) -> list:
        """(layer index, whether a pass of the loop starts here) for every layer run, in execution order."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop
        order = [(i, False) for i in range(a)]
        for _ in range(times):
            order += [(i, i == a) for i in range(a, b)]
        return order + [(i, False) for i in range(b, n)]

    def owner(self, i: int) -> int:
        """Index of the layer whose tensors layer ``i`` runs with (chains are followed)."""
        seen = set()
        while self.layers[i].weights_of is not None:
            if i in seen:
                raise ValueError(f"layer {i}: weights_of forms a cycle")
            seen.add(i)
            i = int(self.layers[i].weights_of)
        return i

    def num_params(self) -> int:
        from vgate.models.hybrid import tensor_shapes
        return sum(math.prod(shape) for shape in tensor_shapes(self).values())

    def to_dict(self) -> dict:
        return asdict(self)


def _zadirax_from_config(cfg: dict, name: str) -> HybridArch:
    """config.json of the Zadirax design: every size and every constant that may differ between
    models of the design is read here; nothing is inferred from a particular checkpoint."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        wo = L.get("weights_of")
        if wo is not None and not (0 <= int(wo) < len(cfg["layers"])) or wo == i:
            raise ValueError(f"layer {i}: weights_of {wo} names no other layer")
        layers.append(LayerSpec(kind=L["type"], mixer=dict(L["mixer"]), mlp=dict(L["mlp"]) if L.get("mlp") else None,
                                weights_of=None if wo is None else int(wo)))
    eos = cfg.get("eos_token_id", 2)
    return HybridArch(name=name, family="zadirax", hidden_size=int(cfg["width"]), vocab_size=int(cfg["vocab"]),
                      layers=tuple(layers), rms_eps=float(cfg["norm"]["eps"]),
                      bos_token_id=int(cfg.get("bos_token_id", 1)),
                      eos_token_ids=tuple(eos) if isinstance(eos, list) else (int(eos),))


def _pozalorn_window(m: dict, qk_norm: str, rotate_values: bool, sink: bool, out_bias: bool) -> dict:
    """Spec of a ``window_attention`` mixer from a Pozalorn attention block."""
    mask = m["mask"]
    return {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
            "scale": float(m["scale"]), "rot": dict(m["rot"]), "window": int(mask["size"]), "pool": int(mask.get("pool") or 0),
            "qk_norm": qk_norm, "rotate_values": rotate_values, "sink": sink, "bias": True, "out_bias": out_bias}


def _pozalorn_mixer(kind: str, m: dict) -> tuple:
    """(key of ``vgate.models.mixers.MIXERS``, its spec) of a Pozalorn layer type. The choices the
    design fixes (which norm, which activations, what is rotated) are written out here, so the mixers
    themselves carry none of them."""
    if kind == "gla":       # gated linear attention: per-channel decay sigmoid(z)^(1 / tau) from a low-rank gate
        return "linear_attention", {"heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                                    "decay": {"kind": "channel", "tau": float(m["tau"])}, "q_scale": float(m["dim"]) ** -0.5,
                                    "in_act": "none", "out_norm": "head", "gate_act": "silu"}
    if kind == "attention":  # window + pooled blocks; whole-projection q / k norm; values rotated by their position
        return "window_attention", _pozalorn_window(m, "all", True, False, False)
    if kind == "parallel":   # sink-softmax window attention beside lightning attention (constant decay per head)
        r = m["right"]
        right = {"heads": int(r["heads"]), "dim": int(r["dim"]), "vdim": int(r["vdim"]),
                 "decay": {"kind": "head", "values": [float(d) for d in r["decay"]]}, "q_scale": 1.0,
                 "in_act": "silu", "out_norm": "all", "gate_act": "sigmoid"}
        if len(right["decay"]["values"]) != right["heads"]:
            raise ValueError("parallel.right: one decay per head")
        return "parallel", {"left": ("window_attention", _pozalorn_window(m["left"], "head", False, True, True)),
                            "right": ("linear_attention", right),
                            "left_scale": float(m["left_scale"]), "right_scale": float(m["right_scale"])}
    raise ValueError(f"Pozalorn has no layer type {kind!r}")


def _pozalorn_from_config(cfg: dict, name: str) -> HybridArch:
    """config.json of the Pozalorn design: sublayers read the stream itself, their outputs are normed
    before they are added, and the next layer reads a learned average over all earlier results."""
    layers = []
    for L in cfg["layers"]:
        kind, spec = _pozalorn_mixer(L["type"], L["mixer"])
        mlp = dict(L["mlp"]) if L.get("mlp") else None
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ValueError(f"Pozalorn feed-forward kind {mlp.get('kind')!r}")
            mlp["act"] = "gelu_tanh"
        layers.append(LayerSpec(kind=kind, mixer=spec, mlp=mlp))
    eos = cfg.get("eos_token_id", 2)
    return HybridArch(name=name, family="pozalorn", hidden_size=int(cfg["width"]), vocab_size=int(cfg["vocab"]),
                      layers=tuple(layers), rms_eps=float(cfg["norm"]["eps"]), bos_token_id=int(cfg.get("bos_token_id", 1)),
                      eos_token_ids=tuple(eos) if isinstance(eos, list) else (int(eos),),
                      arrangement="post_norm", depth_average=True)


def _livitar_mixer(kind: str, m: dict) -> tuple:
    """(key of ``vgate.models.mixers.MIXERS``, its spec) of a Livitar layer type. What the design fixes
    (which norm, which gate, how positions enter) is written out here as options of the general mixers."""
    if kind == "retention":   # constant decay per head, half-split rotary positions on q / k, keys scaled by dim^-1/2
        dec = [float(d) for d in m["decay"]]
        if len(dec) != int(m["heads"]):
            raise ValueError("retention: one decay per head")
        rot = m.get("rot") or {}
        return "linear_attention", {"heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                                    "decay": {"kind": "head", "values": dec}, "q_scale": 1.0, "k_scale": float(m["dim"]) ** -0.5,
                                    "rot": {"dims": int(rot.get("dims", 0)), "base": float(rot.get("base", 10000.0)), "layout": "half"},
                                    "in_act": "none", "out_norm": "head", "norm_weight": False, "gate_act": "silu"}
    if kind in ("attention", "attention_2"):   # full causal softmax attention without rotation, sigmoid output gate
        spec = {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                "scale": float(m["scale"]), "rot": {"dims": 0}, "window": None, "gate": "sigmoid"}
        if kind == "attention":   # per-head temperature; penalty r1 ln(1 + r2 distance)
            spec.update(qk_norm="none", head_temp=True, dist_bias={"kind": "log"})
        else:                     # unit-RMS q / k; query temperature growing with the position; learned bias per distance bucket
            qt = m["q_temp"]
            spec.update(qk_norm="head", qk_norm_weight=False, q_temp={"coef": float(qt["coef"]), "every": int(qt["every"])},
                        dist_bias={"kind": "table", "far": float(m["bias_max"])})
        return "window_attention", spec
    raise ValueError(f"Livitar has no layer type {kind!r}")


def _livitar_mlp(mlp: dict | None) -> dict | None:
    if not mlp:
        return None
    if mlp.get("kind") != "moe":
        raise ValueError(f"Livitar feed-forward kind {mlp.get('kind')!r}")
    r = mlp["router"]
    out = {"kind": "moe", "expert": {"ff": int(mlp["expert"]["ff"]), "act": "silu"},
           "router": {"experts": int(r["experts"]), "top": int(r["top"]), "scale": float(r.get("scale", 1.0)),
                      "score": "softmax", "correction": False}}
    if mlp.get("shared"):
        out["shared"] = {"ff": int(mlp["shared"]["ff"])}
    return out


def _livitar_from_config(cfg: dict, name: str) -> HybridArch:
    """config.json of the Livitar design: pre-norm layers with a tanh norm (no statistics) over several
    copies of the residual stream that every sublayer reads, mixes and writes through learned weights;
    mixers: retention, and two kinds of full causal attention whose positions enter as a bias on the scores."""
    layers = []
    for L in cfg["layers"]:
        kind, spec = _livitar_mixer(L["type"], L["mixer"])
        layers.append(LayerSpec(kind=kind, mixer=spec, mlp=_livitar_mlp(L.get("mlp"))))
    eos = cfg.get("eos_token_id", 2)
    streams = int(cfg.get("streams", 1))
    if streams < 1:
        raise ValueError("streams >= 1")
    return HybridArch(name=name, family="livitar", hidden_size=int(cfg["width"]), vocab_size=int(cfg["vocab"]),
                      layers=tuple(layers), rms_eps=float(cfg["norm"]["eps"]), bos_token_id=int(cfg.get("bos_token_id", 1)),
                      eos_token_ids=tuple(eos) if isinstance(eos, list) else (int(eos),),
                      arrangement="hyper_pre_norm", streams=streams)


def _gefudra_mixer(kind: str, m: dict) -> tuple:
    """(key of ``vgate.models.mixers.MIXERS``, its spec) of a Gefudra layer type. What the design fixes (no
    rotated key part, which gate, which norm, the two score maps) is written out here as options of the mixers."""
    if kind == "latent_attention":   # keys / values from a cached low-rank row; sliding window; sink; sigmoid gate
        return "latent_attention", {"heads": int(m["heads"]), "dim": int(m["dim"]), "rot_dim": 0, "vdim": int(m["vdim"]),
                                    "kv_rank": int(m["kv_rank"]), "q_rank": int(m["q_rank"]), "scale": float(m["scale"]),
                                    "window": int(m["mask"]["size"]), "sink": True, "out_f32": True}
    if kind == "attention":          # two softmax maps per head over the same values, the second subtracted
        rot = m.get("rot") or {}
        return "window_attention", {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
                                    "vdim": int(m["vdim"]), "scale": float(m["scale"]), "window": None,
                                    "rot": {"dims": int(rot.get("dims", 0)), "base": float(rot.get("base", 10000.0)),
                                            "layout": "half"},
                                    "softcap": float(m.get("softcap") or 0.0), "gate": "sigmoid",
                                    "maps": {"count": 2, "init": float(m["diff"])}}
    if kind == "wkv":                # decayed outer-product state with a bonus for the current token, shifted inputs
        return "wkv", {"heads": int(m["heads"]), "dim": int(m["dim"])}
    raise ValueError(f"Gefudra has no layer type {kind!r}")


def _gefudra_from_config(cfg: dict, name: str) -> HybridArch:
    """config.json of the Gefudra design: pre-norm layers (weighted RMS norms) whose results are scaled by
    ``residual_mult`` before they are added, a stretch of layers that runs several times with the same weights
    behind an input matrix over [stream; embedding output], tied output embeddings with a logit scale."""
    layers = []
    for L in cfg["layers"]:
        kind, spec = _gefudra_mixer(L["type"], L["mixer"])
        mlp = L.get("mlp")
        if mlp:
            if mlp.get("kind") != "dense":
                raise ValueError(f"Gefudra feed-forward kind {mlp.get('kind')!r}")
            mlp = {"kind": "dense", "ff": int(mlp["ff"]), "act": "clamped", "limit": float(mlp["limit"])}
        layers.append(LayerSpec(kind=kind, mixer=spec, mlp=mlp or None))
    loop = None
    lp = cfg.get("loop")
    if lp:
        a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
        if not (0 <= a <= b <= len(layers)) or times < 0:
            raise ValueError("loop: 0 <= start <= stop <= layers, times >= 0")
        if b > a:
            loop = (a, b, times)
    eos = cfg.get("eos_token_id", 2)
    return HybridArch(name=name, family="gefudra", hidden_size=int(cfg["width"]), vocab_size=int(cfg["vocab"]),
                      layers=tuple(layers), rms_eps=float(cfg["norm"]["eps"]), bos_token_id=int(cfg.get("bos_token_id", 1)),
                      eos_token_ids=tuple(eos) if isinstance(eos, list) else (int(eos),), arrangement="pre_norm",
                      residual_mult=float(cfg.get("residual_mult", 1.0)), loop=loop,
                      logit_scale=float(cfg.get("logit_scale", 1.0)), tie_embeddings=True)


# config.json "architecture" -> parser of a layered hybrid design
HYBRID_ARCHITECTURES = {"Zadirax": _zadirax_from_config, "Pozalorn": _pozalorn_from_config, "Livitar": _livitar_from_config,
                        "Gefudra": _gefudra_from_config}


def _zadirax_preset(name: str, width: int, vocab: int, pairs: int, heads: int, dim: int, ff: int, experts: int,
                    top: int, expert_ff: int, kv_rank: int, q_rank: int, rot: int, share: bool = False) -> HybridArch:
    """Random-init Zadirax models (benchmarks, tests): ``pairs`` x [general_delta + dense, latent_attention + MoE]."""
    delta = dict(kind="general_delta", mixer={"heads": heads, "dim": dim}, mlp={"kind": "dense", "ff": ff})
    lat = dict(kind="latent_attention",
               mixer={"heads": heads, "dim": dim, "rot_dim": rot, "vdim": dim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "rot": {"base": 10000.0, "dims": rot}, "scale": (dim + rot) ** -0.5},
               mlp={"kind": "moe", "expert": {"ff": expert_ff, "limit": 7.0}, "router": {"experts": experts, "top": top}})
    layers = []
    for i in range(pairs):
        layers.append(LayerSpec(**delta))
        layers.append(LayerSpec(**lat, weights_of=1 if share and i > 0 else None))
    return HybridArch(name=name, family="zadirax", hidden_size=width, vocab_size=vocab, layers=tuple(layers))


def _pozalorn_preset(name: str, width: int, vocab: int, groups: int, heads: int, kv_heads: int, dim: int, ff: int,
                     window: int, pool: int, lin_heads: int | None = None) -> HybridArch:
    """Random-init Pozalorn models (benchmarks, tests): ``groups`` x [gla, attention with pooled blocks,
    sink attention beside lightning attention], each with a dense feed-forward."""
    lh = lin_heads or heads
    rot = {"base": 500000.0, "dims": dim, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    mlp = {"kind": "dense", "ff": ff}
    gla = {"type": "gla", "mixer": {"heads": lh, "dim": dim, "vdim": dim, "tau": 16.0}, "mlp": mlp}
    att = {"type": "attention", "mlp": mlp,
           "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "rot": rot,
                     "mask": {"size": window, "pool": pool}}}
    par = {"type": "parallel", "mlp": mlp,
           "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "rot": rot,
                              "mask": {"size": window}},
                     "right": {"heads": lh, "dim": dim, "vdim": dim,
                               "decay": [math.exp(-(2.0 ** (-8.0 * (i + 1) / lh))) for i in range(lh)]},
                     "left_scale": 1.0, "right_scale": 1.0}}
    cfg = {"width": width, "vocab": vocab, "norm": {"eps": 1e-6}, "layers": [gla, att, par] * groups}
    return _pozalorn_from_config(cfg, name)


def _livitar_preset(name: str, width: int, vocab: int, groups: int, heads: int, kv_heads: int, dim: int, experts: int,
                    top: int, expert_ff: int, shared_ff: int, streams: int = 2, ret_heads: int | None = None,
                    buckets_far: int = 1024) -> HybridArch:
    """Random-init Livitar models (benchmarks, tests): ``groups`` x [retention, attention, attention_2], each
    with a mixture-of-experts feed-forward and a shared expert."""
    rh = ret_heads or heads
    mlp = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "scale": 1.5},
           "shared": {"ff": shared_ff}}
    ret = {"type": "retention", "mlp": mlp,
           "mixer": {"heads": rh, "dim": dim, "vdim": dim, "rot": {"base": 10000.0, "dims": dim},
                     "decay": [1.0 - 2.0 ** (-5.0 - 6.0 * i / max(rh - 1, 1)) for i in range(rh)]}}
    a1 = {"type": "attention", "mlp": mlp,
          "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5}}
    a2 = {"type": "attention_2", "mlp": mlp,
          "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                    "bias_max": buckets_far, "q_temp": {"coef": 0.1, "every": 128}}}
    cfg = {"width": width, "vocab": vocab, "streams": streams, "norm": {"eps": 1e-6}, "layers": [ret, a1, a2] * groups}
    return _livitar_from_config(cfg, name)


def _gefudra_preset(name: str, width: int, vocab: int, groups: int, heads: int, kv_heads: int, dim: int, ff: int,
                    kv_rank: int, q_rank: int, window: int, loop_times: int = 2, wkv_ff: bool = False) -> HybridArch:
    """Random-init Gefudra models (benchmarks, tests): ``groups`` x [latent attention, two-map attention, wkv
    (with a feed-forward only if ``wkv_ff``)], the first group's last two layers looped ``loop_times`` times."""
    mlp = {"kind": "dense", "ff": ff, "limit": 7.0}
    lat = {"type": "latent_attention", "mlp": mlp,
           "mixer": {"heads": heads, "dim": dim, "vdim": dim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": dim ** -0.5,
                     "mask": {"size": window}}}
    att = {"type": "attention", "mlp": mlp,
           "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim // 2, "vdim": dim, "scale": (dim // 2) ** -0.5,
                     "rot": {"base": 10000.0, "dims": dim // 2}, "softcap": 30.0, "diff": 0.5}}
    wkv = {"type": "wkv", "mlp": mlp if wkv_ff else None, "mixer": {"heads": heads, "dim": dim}}
    cfg = {"width": width, "vocab": vocab, "norm": {"eps": 1e-6}, "residual_mult": 0.5, "logit_scale": 1.0,
           "layers": [lat, att, wkv] * groups}
    if loop_times > 0:
        cfg["loop"] = {"start": 1, "stop": 3, "times": loop_times}
    return _gefudra_from_config(cfg, name)


HYBRID_PRESETS = {
    # tests / CPU smoke: odd sizes on purpose (nothing a multiple of the MFMA tile)
    "zadirax-tiny": lambda: _zadirax_preset("zadirax-tiny", 96, 300, 2, 3, 24, 136, 5, 2, 40, 56, 40, 8, share=True),
    # 4-layer slices at the layer sizes of real models, for kernel / step benchmarks beside a transformer of
    # equal width (benchmarks/design_compare.py)
    "zadirax-bench-1024": lambda: _zadirax_preset("zadirax-bench-1024", 1024, 32000, 2, 8, 128, 4096, 8, 2, 2048, 256, 512, 64),
    "zadirax-bench-1536": lambda: _zadirax_preset("zadirax-bench-1536", 1536, 32000, 2, 12, 128, 8960, 16, 4, 2240, 512, 768, 64),
    # tests / CPU smoke: odd sizes on purpose
    "pozalorn-tiny": lambda: _pozalorn_preset("pozalorn-tiny", 88, 300, 1, 4, 2, 24, 136, 21, 5, lin_heads=3),
    # slices at the layer sizes of real models beside a transformer of equal width (benchmarks/design_compare.py)
    "pozalorn-bench-1024": lambda: _pozalorn_preset("pozalorn-bench-1024", 1024, 32000, 1, 8, 2, 128, 4096, 1024, 64),
    "pozalorn-bench-1536": lambda: _pozalorn_preset("pozalorn-bench-1536", 1536, 32000, 1, 12, 2, 128, 8960, 1024, 64),
    # tests / CPU smoke: odd sizes on purpose
    "livitar-tiny": lambda: _livitar_preset("livitar-tiny", 88, 300, 1, 4, 2, 24, 5, 2, 40, 56, streams=3, ret_heads=3, buckets_far=50),
    # slices at the layer sizes of real models beside a transformer of equal width (benchmarks/design_compare.py)
    # (the chosen experts and the shared one together are as wide as the dense feed-forward of the other bench presets)
    "livitar-bench-1024": lambda: _livitar_preset("livitar-bench-1024", 1024, 32000, 1, 8, 2, 128, 8, 2, 1024, 2048),
    "livitar-bench-1536": lambda: _livitar_preset("livitar-bench-1536", 1536, 32000, 1, 12, 2, 128, 16, 4, 1792, 1792),
    # tests / CPU smoke: odd sizes on purpose
    "gefudra-tiny": lambda: _gefudra_preset("gefudra-tiny", 88, 300, 1, 4, 2, 24, 136, 40, 56, 21),
    # slices at the layer sizes of real models beside a transformer of equal width (benchmarks/design_compare.py):
    # three layers with a feed-forward each, as in the other designs' bench presets; the loop runs once (its input
    # matrix is applied, no layer runs twice)
    "gefudra-bench-1024": lambda: _gefudra_preset("gefudra-bench-1024", 1024, 32000, 1, 8, 2, 128, 4096, 256, 512, 1024,
                                                  loop_times=1, wkv_ff=True),
    "gefudra-bench-1536": lambda: _gefudra_preset("gefudra-bench-1536", 1536, 32000, 1, 12, 2, 128, 8960, 512, 768, 1024,
                                                  loop_times=1, wkv_ff=True),
    # layer sizes of a ~1.5B model (the width, head size, feed-forward and vocabulary of qwen2.5-1.5b)
    "zadirax-1.5b": lambda: _zadirax_preset("zadirax-1.5b", 1536, 151936, 14, 12, 128, 8960, 32, 4, 2240, 512, 768, 64),
}


def resolve_arch(model_id: str, overrides: dict | None = None):
    """Resolve a model id / path to its architecture."""
    p = Path(os.path.expanduser(model_id))
    arch = None
    if p.is_dir() and (p / "config.json").exists():
        cfg = json.loads((p / "config.json").read_text())
        parse = HYBRID_ARCHITECTURES.get(cfg.get("architecture"))
        arch = parse(cfg, p.name) if parse else _from_hf_config(cfg, p.name)
    else:
        key = model_id.lower().split("/")[-1]
        key = key.replace("-instruct", "").replace("-awq", "").replace("_", "-")
        if key in HYBRID_PRESETS:
            arch = HYBRID_PRESETS[key]()
        for alias, preset in _ALIASES:
            if arch is not None:
                break
            if alias in key:
                arch = PRESETS[preset]
                break
    if arch is None:
        raise ValueError(f"unknown model '{model_id}': pass a directory with config.json or one of "
                         f"{sorted(PRESETS) + sorted(HYBRID_PRESETS)}")
    if overrides:
        arch = replace(arch, **overrides)
    return arch
