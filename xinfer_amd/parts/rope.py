"""Rotary position encoding: the tables the attention kernel reads.

inv_freq[i] = 1f32 / (f32)(theta^(2i/rot)) with the power in float64, angle =
(f32)p * inv_freq[i] in float32, cos/sin of that angle (reference:
/root/reference/src/models/layers/rotary_emb.rs:47-61).  The reference stores the
tables in the model dtype; here they stay float32 in both precisions, so rotation
angles are 32-bit everywhere.  The rotation itself is fused into the kernel that also
norms q/k and writes the cache (`kernels.qk_norm_rope_kv`).

A `scaling` parameter (config.json's rope_scaling) changes the frequencies, and for YaRN also
scales cos and sin, as the reference's ScalingRotaryEmbedding does (rotary_emb.rs:126-415,
482-540); the table's rows are the positions the model can encode.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from ..config.spec import PartSpec
from .base import PositionEncoding, register_position_encoding


@register_position_encoding("rope")
class RotaryEmbedding(PositionEncoding):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.head_dim = int(spec["head_dim"])
        self.rotary_dim = int(spec.get("rotary_dim", self.head_dim))
        self.theta = float(spec["theta"])
        self.max_positions = int(spec["max_positions"])
        self.interleaved = bool(spec.get("interleaved", False))
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.cos = self.sin = None

    def load(self, store, prefix, device) -> None:
        scaling = self.spec.get("scaling")
        key = (self.rotary_dim, self.theta, self.max_positions, str(torch.device(device)),
               tuple(sorted(scaling.items())) if scaling else None)
        if key not in _TABLES:
            inv_freq, mscale = scaled_inv_freq(self.theta, self.rotary_dim, scaling)
            pos = torch.arange(self.max_positions, dtype=torch.float32)
            ang = pos[:, None] * torch.from_numpy(inv_freq)[None, :]          # float32 product
            cos, sin = ang.cos(), ang.sin()
            if mscale != 1.0:
                cos, sin = cos * mscale, sin * mscale
            _TABLES[key] = (cos.contiguous().to(device), sin.contiguous().to(device))
        self.cos, self.sin = _TABLES[key]


def _default_inv_freq(theta: float, rot: int) -> np.ndarray:
    """1f32 / (f32)(theta^(i/rot)) for i = 0, 2, ..: the power in float64, the division in float32
    (calculate_default_inv_freq, rotary_emb.rs:116-121)."""
    powers = np.power(np.float64(theta), np.arange(0, rot, 2, dtype=np.float64) / rot).astype(np.float32)
    return (np.float32(1.0) / powers).astype(np.float32)


def scaled_inv_freq(theta: float, rot: int, scaling) -> "tuple[np.ndarray, float]":
    """(inv_freq float32 [rot / 2], factor on cos and sin) for a `scaling` of the kinds of the
    reference (rotary_emb.rs:172-401), with its float32 and float64 roles.  `scaling`: a mapping
    with `kind`, `original` (the length the model was trained at) and the kind's numbers."""
    f32 = np.float32
    if not scaling or scaling["kind"] == "default":
        return _default_inv_freq(theta, rot), 1.0
    kind, orig = scaling["kind"], float(scaling["original"])
    if kind == "linear":                                    # rotary_emb.rs:172-206: a float32 product with 1 / factor
        return (_default_inv_freq(theta, rot) * f32(1.0 / float(scaling["factor"]))).astype(f32), 1.0
    if kind == "llama3":                                    # rotary_emb.rs:208-282, all float32
        factor, low, high = f32(scaling["factor"]), f32(scaling["low_freq_factor"]), f32(scaling["high_freq_factor"])
        low_wavelen, high_wavelen = f32(orig / float(scaling["low_freq_factor"])), f32(orig / float(scaling["high_freq_factor"]))
        out = []
        for freq in _default_inv_freq(theta, rot):
            wavelen = f32(2.0) * f32(math.pi) / freq
            if wavelen < high_wavelen:
                out.append(freq)
            elif wavelen > low_wavelen:
                out.append(freq / factor)
            else:
                smooth = (f32(orig) / wavelen - low) / (high - low)
                out.append((f32(1.0) - smooth) * freq / factor + smooth * freq)
        return np.asarray(out, dtype=f32), 1.0
    if kind == "dynamic":                                   # rotary_emb.rs:284-335: a larger base, in float64
        power = rot / (rot - 2.0)
        if scaling.get("alpha") is not None:
            base = (theta * float(scaling["alpha"])) ** power
        else:
            factor = float(scaling["factor"])
            max_len = float(int(orig * factor))
            base = (theta * ((factor * max_len / orig) - (factor - 1.0))) ** power
        return _default_inv_freq(base, rot), 1.0
    if kind == "yarn":                                      # rotary_emb.rs:482-540, all float32
        factor, base = f32(scaling["factor"]), f32(theta)
        steps = np.arange(0, rot, 2, dtype=f32) / f32(rot)
        powers = np.power(base, steps).astype(f32)
        extra = (f32(1.0) / powers).astype(f32)                               # the frequencies as they are
        inter = (f32(1.0) / (factor * powers)).astype(f32)                    # and stretched by the factor

        def correction_dim(rotations: float) -> np.float32:
            return (f32(rot) * np.log(f32(orig) / (f32(rotations) * f32(2.0) * f32(math.pi)))) / (f32(2.0) * np.log(base))

        low = max(float(np.floor(correction_dim(scaling["beta_fast"]))), 0.0)
        high = min(float(np.ceil(correction_dim(scaling["beta_slow"]))), rot - 1.0)
        if low == high:
            high += 0.001
        ramp = np.clip((np.arange(rot // 2, dtype=f32) - f32(low)) * f32(1.0 / (high - low)), 0.0, 1.0).astype(f32)
        mask = ((f32(1.0) - ramp) * f32(scaling["extrapolation_factor"])).astype(f32)
        inv = (inter * (f32(1.0) - mask) + extra * mask).astype(f32)
        mscale = f32(1.0) if factor <= 1.0 else f32(0.1) * f32(1.0) * np.log(factor) + f32(1.0)
        return inv, float(f32(mscale * f32(scaling["attn_factor"])))
    raise ValueError(f"Unknown rope_type: {kind}")


# layers with the same rotary parameters share one pair of tables per device
_TABLES = {}
