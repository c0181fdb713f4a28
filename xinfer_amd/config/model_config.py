"""Typed model configuration read from an architecture's own config.json keys.

The reference keeps one serde struct with optional fields for every architecture
(/root/reference/src/utils/config.rs:277-330).  Here each architecture has its own
typed class, and the class knows how to describe itself as an architecture-neutral
`ModelSpec` (see `spec.py`), which is what the rest of the engine consumes.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any, Dict, List, Optional, Tuple


class ConfigError(ValueError):
    """Raised for a config.json that the engine cannot run."""


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"Model file(s) not found: no config.json in {model_dir!r}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            raw = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from e
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return raw


def architecture_name(raw: Dict[str, Any]) -> str:
    """The reference insists on exactly one entry in `architectures`
    (/root/reference/src/core/engine.rs:166-169)."""
    archs = raw.get("architectures")
    if not isinstance(archs, list) or len(archs) != 1 or not isinstance(archs[0], str):
        raise ConfigError(
            f"config.json must name exactly one architecture in 'architectures', got {archs!r}")
    return archs[0]


def _require(raw: Dict[str, Any], key: str, typ, where: str):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"{where}: required key {key!r} is missing")
    return _typed(raw[key], key, typ, where)


def _typed(v, key: str, typ, where: str):
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and float(v).is_integer():
                return int(v)
            raise ConfigError(f"{where}: key {key!r} must be an integer, got {v!r}")
        return v
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: key {key!r} must be a number, got {v!r}")
        return float(v)
    if typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: key {key!r} must be true or false, got {v!r}")
        return v
    if typ is str:
        if not isinstance(v, str):
            raise ConfigError(f"{where}: key {key!r} must be a string, got {v!r}")
        return v
    raise TypeError(typ)


@dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense (`Qwen3ForCausalLM`).

    Required keys follow the reference's `Config` (config.rs:277-330): the head
    counts, hidden size, layer count, eps, max positions and activation.  Optional
    keys and their defaults: `head_dim = hidden_size / num_attention_heads`
    (attention.rs:446), `rope_theta = 10000` (rotary_emb.rs:49),
    `tie_word_embeddings = false` (qwen3.rs:200-209), `attention_bias`
    ("load the bias if the tensor exists" in the reference; here an explicit flag,
    default false as in Qwen3 checkpoints), `sliding_window` (passed to every
    layer when present, qwen3.rs:46) and `layer_types`, which restricts the window
    to the layers it names "sliding_attention".
    """
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    hidden_act: str = "silu"
    sliding_window: Optional[int] = None
    layer_types: Optional[Tuple[str, ...]] = None
    eos_token_id: Optional[Tuple[int, ...]] = None
    bos_token_id: Optional[int] = None
    architecture: str = "Qwen3ForCausalLM"

    # ---- construction -------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "Qwen3Config":
        h = _require(raw, "hidden_size", int, where)
        nq = _require(raw, "num_attention_heads", int, where)
        nkv = _require(raw, "num_key_value_heads", int, where)
        if nq <= 0 or nkv <= 0 or h <= 0:
            raise ConfigError(f"{where}: sizes must be positive")
        if raw.get("head_dim") is not None:
            d = _typed(raw["head_dim"], "head_dim", int, where)
        else:
            if h % nq:
                raise ConfigError(
                    f"{where}: head_dim is absent and hidden_size {h} is not a multiple of "
                    f"num_attention_heads {nq}")
            d = h // nq
        if raw.get("vocab_size") is None:
            # the reference asserts this for safetensors models (others.rs:327-330)
            raise ConfigError(f"{where}: required key 'vocab_size' is missing")
        eos = raw.get("eos_token_id")
        if eos is None:
            eos_t = None
        elif isinstance(eos, list):
            eos_t = tuple(_typed(e, "eos_token_id", int, where) for e in eos)
        else:
            eos_t = (_typed(eos, "eos_token_id", int, where),)
        lt = raw.get("layer_types")
        if lt is not None:
            if not isinstance(lt, list) or not all(isinstance(s, str) for s in lt):
                raise ConfigError(f"{where}: 'layer_types' must be a list of strings")
            lt = tuple(lt)
        sw = raw.get("sliding_window")
        if sw is not None:
            sw = _typed(sw, "sliding_window", int, where)
        scaling = raw.get("rope_scaling", raw.get("rope_parameters"))
        if scaling is not None:
            kind = None
            if isinstance(scaling, dict):
                kind = scaling.get("rope_type", scaling.get("type"))
            if kind not in (None, "default"):
                raise ConfigError(
                    f"{where}: rope_scaling of type {kind!r} is not supported (plain RoPE only)")
        cfg = cls(
            vocab_size=_typed(raw["vocab_size"], "vocab_size", int, where),
            hidden_size=h,
            intermediate_size=_require(raw, "intermediate_size", int, where),
            num_hidden_layers=_require(raw, "num_hidden_layers", int, where),
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=d,
            max_position_embeddings=_require(raw, "max_position_embeddings", int, where),
            rms_norm_eps=_require(raw, "rms_norm_eps", float, where),
            rope_theta=_typed(raw.get("rope_theta", 10000.0) if raw.get("rope_theta") is not None
                              else 10000.0, "rope_theta", float, where),
            tie_word_embeddings=_typed(raw["tie_word_embeddings"], "tie_word_embeddings", bool, where)
            if raw.get("tie_word_embeddings") is not None else False,
            attention_bias=_typed(raw["attention_bias"], "attention_bias", bool, where)
            if raw.get("attention_bias") is not None else False,
            hidden_act=_typed(raw.get("hidden_act", raw.get("hidden_activation", "silu")),
                              "hidden_act", str, where),
            sliding_window=sw,
            layer_types=lt,
            eos_token_id=eos_t,
            bos_token_id=_typed(raw["bos_token_id"], "bos_token_id", int, where)
            if raw.get("bos_token_id") is not None else None,
            architecture=raw.get("architectures", ["Qwen3ForCausalLM"])[0],
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{where}: {name} must be positive, got {getattr(self, name)}")
        if self.num_hidden_layers < 0:
            raise ConfigError(f"{where}: num_hidden_layers must not be negative")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"{where}: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for rotary pairs")
        if self.hidden_act != "silu":
            raise ConfigError(
                f"{where}: hidden_act {self.hidden_act!r} is not supported (silu only)")
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError(f"{where}: rms_norm_eps must not be negative")
        if self.rope_theta <= 0.0:
            raise ConfigError(f"{where}: rope_theta must be positive")
        if self.sliding_window is not None and self.sliding_window <= 0:
            raise ConfigError(f"{where}: sliding_window must be positive or null")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError(
                    f"{where}: layer_types has {len(self.layer_types)} entries for "
                    f"{self.num_hidden_layers} layers")
            for t in self.layer_types:
                if t not in ("full_attention", "sliding_attention"):
                    raise ConfigError(f"{where}: unknown layer type {t!r}")
                if t == "sliding_attention" and self.sliding_window is None:
                    raise ConfigError(
                        f"{where}: layer_types names sliding_attention but sliding_window is null")

    # ---- serialisation ------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architectures": [self.architecture], "model_type": "qwen3"}
        for f in fields(self):
            if f.name == "architecture":
                continue
            v = getattr(self, f.name)
            if isinstance(v, tuple):
                v = list(v)
            if f.name == "eos_token_id" and v is not None and len(v) == 1:
                v = v[0]
            out[f.name] = v
        return out

    def window_of_layer(self, i: int) -> Optional[int]:
        """Window (number of keys a query sees, itself included) of layer `i`, or None."""
        if self.sliding_window is None:
            return None
        if self.layer_types is None:
            return self.sliding_window
        return self.sliding_window if self.layer_types[i] == "sliding_attention" else None
