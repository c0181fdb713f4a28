"""Typed model configuration read from an architecture's own config.json keys.

The reference keeps one serde struct with optional fields for every architecture
(/root/reference/src/utils/config.rs:277-330).  Here each architecture has its own
typed class, and the class knows how to describe itself as an architecture-neutral
`ModelSpec` (see `spec.py`), which is what the rest of the engine consumes.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields
from typing import Any, Dict, Optional, Tuple


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


ROPE_SCALING_KINDS = ("default", "linear", "llama3", "dynamic", "yarn")


@dataclass(frozen=True)
class RopeScaling:
    """config.json's `rope_scaling` (or `rope_parameters`), typed.  The kinds and their keys are
    those of the reference's ScalingRotaryEmbedding::new
    (/root/reference/src/models/layers/rotary_emb.rs:126-415): "linear" (factor), "llama3"
    (factor, low_freq_factor, high_freq_factor), "dynamic" (alpha, or factor), "yarn" (factor;
    beta_fast 32, beta_slow 1, extrapolation_factor 1, attn_factor 1 unless given); "default" is
    plain RoPE.  `original_max_position_embeddings` as the file gives it, or None."""
    kind: str
    factor: Optional[float] = None
    original_max_position_embeddings: Optional[float] = None
    low_freq_factor: Optional[float] = None
    high_freq_factor: Optional[float] = None
    alpha: Optional[float] = None
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    extrapolation_factor: float = 1.0
    attn_factor: float = 1.0

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> Optional["RopeScaling"]:
        if raw is None:
            return None
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: 'rope_scaling' must be an object")
        kind = raw.get("rope_type", raw.get("type"))       # rotary_emb.rs:146-150
        if kind is None and "rope_theta" in raw and len(raw) == 1:
            return None                                        # `rope_parameters` that only repeats the base
        if not isinstance(kind, str):
            raise ConfigError(f"{where}: rope_scaling needs a string 'rope_type'")
        if kind not in ROPE_SCALING_KINDS:
            raise ConfigError(f"{where}: Unknown rope_type: {kind} (known: {', '.join(ROPE_SCALING_KINDS)})")

        def num(key, default=None):
            v = raw.get(key)
            return default if v is None else _typed(v, f"rope_scaling.{key}", float, where)

        rs = cls(kind=kind, factor=num("factor"),
                 original_max_position_embeddings=num("original_max_position_embeddings"),
                 low_freq_factor=num("low_freq_factor"), high_freq_factor=num("high_freq_factor"),
                 alpha=num("alpha"), beta_fast=num("beta_fast", 32.0), beta_slow=num("beta_slow", 1.0),
                 extrapolation_factor=num("extrapolation_factor", 1.0), attn_factor=num("attn_factor", 1.0))
        if kind == "linear" and rs.factor is None:
            raise ConfigError(f"{where}: Linear rope_type requires factor to be set")
        if kind == "llama3" and None in (rs.factor, rs.low_freq_factor, rs.high_freq_factor):
            raise ConfigError(f"{where}: Llama3 rope_type requires factor, low_freq_factor, high_freq_factor to be set")
        if kind == "llama3" and rs.high_freq_factor == rs.low_freq_factor:
            raise ConfigError(f"{where}: llama3 rope_type needs high_freq_factor and low_freq_factor to differ")
        if kind == "dynamic" and rs.alpha is None and rs.factor is None:
            raise ConfigError(f"{where}: Dynamic rope_type requires either alpha or factor to be set")
        if kind == "yarn" and rs.factor is None:
            raise ConfigError(f"{where}: yarn rope_type requires factor to be set")
        for key in ("factor", "alpha", "original_max_position_embeddings"):
            v = getattr(rs, key)
            if v is not None and not v > 0.0:
                raise ConfigError(f"{where}: rope_scaling.{key} must be positive, got {v}")
        return rs

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"rope_type": self.kind}
        defaults = RopeScaling(self.kind)
        for f in fields(self):
            v = getattr(self, f.name)
            if f.name != "kind" and v is not None and v != getattr(defaults, f.name):
                out[f.name] = v
        return out

    def original_positions(self, max_position_embeddings: int) -> float:
        """The length the model was trained at: as given, else max / factor, else max (rotary_emb.rs:152-166)."""
        if self.original_max_position_embeddings is not None:
            return self.original_max_position_embeddings
        if self.factor is not None:
            return max_position_embeddings / self.factor
        return float(max_position_embeddings)


def derive_yarn_scaling(factor: float, max_position_embeddings: int) -> RopeScaling:
    """The `rope_scaling` that the reference's --yarn-scaling-factor option puts in place of the
    file's (/root/reference/src/utils/mod.rs:806-871): YaRN over the file's length, beta_fast grown
    with sqrt(factor / 4) and the extrapolation factor a little above 1 for large factors."""
    factor = max(float(factor), 1.0)
    beta_fast = 32.0 if factor <= 4.0 else 32.0 * (factor / 4.0) ** 0.5
    extrapolation = 1.0 + 0.05 * (factor - 8.0) ** 0.5 if factor > 8.0 else 1.0
    return RopeScaling("yarn", factor=factor, original_max_position_embeddings=float(max_position_embeddings),
                       beta_fast=beta_fast, beta_slow=1.0, extrapolation_factor=extrapolation, attn_factor=1.0)


@dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense (`Qwen3ForCausalLM`).

    Required keys follow the reference's `Config` (config.rs:277-330): the head
    counts, hidden size, layer count, eps, max positions and activation.  Optional
    keys and their defaults: `head_dim = hidden_size / num_attention_heads`
    (attention.rs:446), `rope_theta = 10000` (rotary_emb.rs:49),
    `tie_word_embeddings = false` (qwen3.rs:200-209), `qkv_bias` or else `attention_bias`
    (when neither is given the reference loads the q, k and v biases if the checkpoint has them,
    attention.rs:472-476 and 388-399: here None, decided by the tensors' names when a
    checkpoint is read and off for random weights), `sliding_window` (passed to every
    layer when present, qwen3.rs:46) and `layer_types`, which restricts the window
    to the layers it names "sliding_attention"; `rope_scaling` (see `RopeScaling`) and
    `partial_rotary_factor` (the first int(factor * head_dim) dims of a head are rotated,
    rotary_emb.rs:138-141).
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
    attention_bias: Optional[bool] = None
    hidden_act: str = "silu"
    sliding_window: Optional[int] = None
    layer_types: Optional[Tuple[str, ...]] = None
    eos_token_id: Optional[Tuple[int, ...]] = None
    bos_token_id: Optional[int] = None
    rope_scaling: Optional[RopeScaling] = None
    partial_rotary_factor: Optional[float] = None
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
        # what the reference's attention reads of a configuration and this engine does not compute
        # (attention.rs:477-481, 698): refused rather than left out of the result
        if raw.get("attn_logit_softcapping") is not None:
            raise ConfigError(f"{where}: attn_logit_softcapping is not supported")
        if raw.get("attn_output_gate"):
            raise ConfigError(f"{where}: attn_output_gate is not supported")
        scaling = RopeScaling.from_dict(raw.get("rope_scaling", raw.get("rope_parameters")), where)
        prf = raw.get("partial_rotary_factor")
        if prf is not None:
            prf = _typed(prf, "partial_rotary_factor", float, where)
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
            attention_bias=_typed(raw["qkv_bias"], "qkv_bias", bool, where) if raw.get("qkv_bias") is not None
            else _typed(raw["attention_bias"], "attention_bias", bool, where) if raw.get("attention_bias") is not None
            else None,
            hidden_act=_typed(raw.get("hidden_act", raw.get("hidden_activation", "silu")),
                              "hidden_act", str, where),
            sliding_window=sw,
            layer_types=lt,
            eos_token_id=eos_t,
            bos_token_id=_typed(raw["bos_token_id"], "bos_token_id", int, where)
            if raw.get("bos_token_id") is not None else None,
            rope_scaling=scaling,
            partial_rotary_factor=prf,
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
        if self.partial_rotary_factor is not None:
            if not (0.0 < self.partial_rotary_factor <= 1.0):
                raise ConfigError(f"{where}: partial_rotary_factor must be in (0, 1], got {self.partial_rotary_factor}")
            if self.rotary_dim < 2 or self.rotary_dim % 2:
                raise ConfigError(f"{where}: partial_rotary_factor {self.partial_rotary_factor} of head_dim "
                                  f"{self.head_dim} gives {self.rotary_dim} rotated dims; an even number of at least 2 is needed")
        if self.rope_scaling is not None and self.rope_scaling.kind == "dynamic" and self.rotary_dim <= 2:
            raise ConfigError(f"{where}: dynamic rope scaling needs more than 2 rotated dims")
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
            if f.name in ("rope_scaling", "partial_rotary_factor") and v is None:
                continue
            if isinstance(v, RopeScaling):
                v = v.to_dict()
            if isinstance(v, tuple):
                v = list(v)
            if f.name == "eos_token_id" and v is not None and len(v) == 1:
                v = v[0]
            out[f.name] = v
        return out

    @property
    def rotary_dim(self) -> int:
        """Dims of a head that are rotated (rotary_emb.rs:138-141)."""
        if self.partial_rotary_factor is None:
            return self.head_dim
        return int(self.partial_rotary_factor * self.head_dim)

    @property
    def positions(self) -> int:
        """Positions the model can encode.  YaRN over a given original length reaches
        round(original * factor) if that is more than max_position_embeddings
        (effective_max_position_embeddings, /root/reference/src/utils/mod.rs:873-897)."""
        rs = self.rope_scaling
        if (rs is not None and rs.kind == "yarn" and rs.factor is not None and rs.factor > 1.0
                and rs.original_max_position_embeddings is not None):
            return max(self.max_position_embeddings, int(round(rs.original_max_position_embeddings * rs.factor)))
        return self.max_position_embeddings

    def with_yarn_scaling(self, factor: float) -> "Qwen3Config":
        """The configuration under the --yarn-scaling-factor option: YaRN over this file's length,
        in place of whatever rope_scaling the file has (apply_runtime_rope_overrides,
        /root/reference/src/utils/mod.rs:862-869)."""
        import dataclasses
        out = dataclasses.replace(self, rope_scaling=derive_yarn_scaling(factor, self.max_position_embeddings))
        out.validate("config.json with yarn_scaling_factor")
        return out

    def window_of_layer(self, i: int) -> Optional[int]:
        """Window (number of keys a query sees, itself included) of layer `i`, or None."""
        if self.sliding_window is None:
            return None
        if self.layer_types is None:
            return self.sliding_window
        return self.sliding_window if self.layer_types[i] == "sliding_attention" else None
