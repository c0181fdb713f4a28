"""Rotary position encoding: the tables the attention kernel reads.

inv_freq[i] = 1f32 / (f32)(theta^(2i/rot)) with the power in float64, angle =
(f32)p * inv_freq[i] in float32, cos/sin of that angle (reference:
/root/reference/src/models/layers/rotary_emb.rs:47-61).  The reference stores the
tables in the model dtype; here they stay float32 in both precisions, so rotation
angles are 32-bit everywhere.  The rotation itself is fused into the kernel that also
norms q/k and writes the cache (`kernels.qk_norm_rope_kv`).
"""
from __future__ import annotations

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
        key = (self.rotary_dim, self.theta, self.max_positions, str(torch.device(device)))
        if key not in _TABLES:
            idx = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
            powers = (torch.tensor(self.theta, dtype=torch.float64) ** (idx / self.rotary_dim))
            inv_freq = 1.0 / powers.to(torch.float32)       # float32 division, as in the reference
            pos = torch.arange(self.max_positions, dtype=torch.float32)
            ang = pos[:, None] * inv_freq[None, :]          # float32 product
            _TABLES[key] = (ang.cos().contiguous().to(device), ang.sin().contiguous().to(device))
        self.cos, self.sin = _TABLES[key]


# layers with the same rotary parameters share one pair of tables per device
_TABLES = {}
