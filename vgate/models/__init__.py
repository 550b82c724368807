"""Model families and the registry that maps an architecture to its model class."""
from __future__ import annotations

# family (ModelArch.family / HybridArch.family) -> model class, imported on first use
TRANSFORMER_FAMILIES = {"qwen2", "llama"}   # vgate.models.transformer.DecoderModel
HYBRID_FAMILIES = {"zadirax", "pozalorn", "livitar", "gefudra"}   # vgate.models.hybrid.HybridModel (layered: mixers + feed-forwards)


def build_model(arch, device, tp=None, quantization=None, seed: int = 0, weights_path: str | None = None,
                max_model_len: int = 4096, dtype: str = "bfloat16"):
    """Instantiate the model class of ``arch.family`` (weights loaded from ``weights_path`` or
    random-initialised from ``seed``)."""
    dtype = {"auto": "bfloat16", "bf16": "bfloat16", "fp32": "float32"}.get(dtype, dtype)
    if arch.family in TRANSFORMER_FAMILIES:
        from vgate.models.transformer import DecoderModel
        if dtype == "float32":
            raise ValueError(f"the {arch.family} family runs in bfloat16 only (dtype {dtype!r} asked)")
        return DecoderModel(arch, device, tp, quantization, seed, weights_path, max_model_len)
    if arch.family in HYBRID_FAMILIES:
        from vgate.models.hybrid import HybridModel
        return HybridModel(arch, device, tp, quantization, seed, weights_path, max_model_len, dtype=dtype)
    raise ValueError(f"no model class for family {arch.family!r} (known: "
                     f"{sorted(TRANSFORMER_FAMILIES | HYBRID_FAMILIES)})")
