"""From a model folder (or a typed config and a weight store) to a loaded model."""
from __future__ import annotations

from typing import Optional

import torch

from ..models import family_of, load_config
from ..weights.store import SafetensorsStore, WeightStore
from .model import CausalLM

_DTYPES = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16, "f32": torch.float32,
           "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    """The reference takes --dtype f16|bf16|f32 (/root/reference/src/utils/mod.rs:2479-2486);
    float16 is not built here."""
    if hasattr(name, "value") and isinstance(getattr(name, "value"), str):      # the DType enum
        name = name.value
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype {name} is not supported (bfloat16 or float32)")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype {name!r} is not supported (bf16/bfloat16 or f32/float32)") from None


def load_model(model_dir: str, dtype, device="cuda:0", yarn_scaling_factor: Optional[float] = None) -> CausalLM:
    """`yarn_scaling_factor`: stretch the model's positions by this factor with YaRN, whatever the
    folder's config.json says about rope scaling (the reference's --yarn-scaling-factor)."""
    fam, cfg = load_config(model_dir)
    if yarn_scaling_factor is not None:
        if not hasattr(cfg, "with_yarn_scaling"):
            raise ValueError(f"yarn_scaling_factor: the {fam.name} family has no rope scaling to set")
        cfg = cfg.with_yarn_scaling(float(yarn_scaling_factor))
    store = SafetensorsStore(model_dir)
    try:
        return build_model(cfg, store, dtype, device)
    finally:
        store.close()


def build_model(config, store: WeightStore, dtype, device="cuda:0") -> CausalLM:
    fam = family_of(config.architecture)
    model = CausalLM(fam.spec(config, store.names()), parse_dtype(dtype))
    model.config = config
    return model.load(store, device)
