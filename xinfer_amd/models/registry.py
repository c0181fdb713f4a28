"""One registry from an architecture's name to its model family.

The reference maps `architectures[0]` to a `ModelType` in `get_arch_rope`
(/root/reference/src/utils/mod.rs:2297-2477) and builds the model with the
`build_model!` macro (/root/reference/src/core/mod.rs:130-150).  Here a family is
a config class plus a function that turns the typed config into a `ModelSpec`;
everything after that is architecture-neutral.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Sequence

from ..config.model_config import ConfigError, architecture_name, read_config_json
from ..config.spec import ModelSpec


@dataclass(frozen=True)
class ModelFamily:
    name: str
    config_class: Any                       # has from_dict(raw, where) and to_dict()
    build_spec: Callable[[Any], ModelSpec]  # typed config -> ModelSpec
    # (typed config, names of the tensors a checkpoint holds) -> ModelSpec, for a family whose
    # checkpoints come in more than one naming; None: `build_spec` whatever the names
    build_spec_for: Optional[Callable[[Any, Sequence[str]], ModelSpec]] = None
    # the chat template (jinja) of a model folder whose tokenizer_config.json carries none
    chat_template: Optional[str] = None

    def spec(self, config, tensor_names: Optional[Sequence[str]] = None) -> ModelSpec:
        if tensor_names is not None and self.build_spec_for is not None:
            return self.build_spec_for(config, tensor_names)
        return self.build_spec(config)


_FAMILIES: Dict[str, ModelFamily] = {}


def register_architecture(arch_name: str, family: ModelFamily) -> None:
    _FAMILIES[arch_name] = family


def registered_architectures():
    return sorted(_FAMILIES)


def family_of(arch_name: str) -> ModelFamily:
    try:
        return _FAMILIES[arch_name]
    except KeyError:
        raise ConfigError(
            f"Unsupported architecture: {arch_name!r} (supported: {', '.join(registered_architectures())})"
        ) from None


def load_config(model_dir: str):
    """Read config.json and return (family, typed config)."""
    raw = read_config_json(model_dir)
    fam = family_of(architecture_name(raw))
    return fam, fam.config_class.from_dict(raw, where=f"{model_dir}/config.json")


def config_from_dict(raw: Dict[str, Any]):
    fam = family_of(architecture_name(raw))
    return fam, fam.config_class.from_dict(raw)
