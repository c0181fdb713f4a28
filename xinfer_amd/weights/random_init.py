"""Random-weights mode: writes a model folder from a configuration and a seed.

The folder holds config.json (the architecture's own keys) and model.safetensors with
every tensor the architecture's parts declare: linear weights ~ N(0, linear_std), norm
weights ~ 1 + N(0, norm_std), rounded to `dtype`.  The reference has no such mode; it is
what tests and benchmarks run on, there being no checkpoints without a network.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Union

import torch

from .safetensors_io import write_safetensors
from .store import RandomStore


def random_store_for(config, seed: int, linear_std: float = 0.02, norm_std: float = 0.1,
                     dtype: torch.dtype = torch.bfloat16) -> RandomStore:
    """A RandomStore holding every tensor of the model that `config` describes."""
    from ..engine.model import CausalLM
    from ..models import family_of
    fam = family_of(config.architecture)
    spec = fam.build_spec(config)
    return RandomStore(CausalLM.declare(spec), seed, linear_std, norm_std, dtype)


def write_random_model(model_dir: str, config: Union[Dict[str, Any], Any], seed: int,
                       linear_std: float = 0.02, norm_std: float = 0.1,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """`config` is a typed config or a config.json dictionary.  Returns `model_dir`."""
    from ..models import config_from_dict
    if isinstance(config, dict):
        _, config = config_from_dict(config)
    store = random_store_for(config, seed, linear_std, norm_std, dtype)
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=1)
    # the values are the same wherever they are made; the GPU, if there is one, makes large tables faster
    device = "cuda" if torch.cuda.is_available() else "cpu"
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      ((name, store.get(name, None, device).cpu()) for name in store.names()))
    return model_dir
