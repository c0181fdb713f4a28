"""RMSNorm on the float32 residual stream, fused with the residual add.

out = s * rsqrt(mean(s^2) + eps) * w with s = resid (+ add), everything in float32 and
one rounding to the output type (reference: NormX::forward and forward_add,
/root/reference/src/models/layers/others.rs:22-62; weight kept in float32,
/root/reference/src/models/qwen3.rs:83).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    foldable = True      # the products around it can carry it (parts.base.Folded)

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.dim = int(spec["dim"])
        self.eps = float(spec["eps"])
        self.weight: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        return [TensorDecl(f"{prefix}.weight" if "name" not in spec.params else spec["name"],
                           (int(spec["dim"]),), "norm")]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        name = self.spec.get("name") or f"{prefix}.weight"
        self.weight = store.get(name, torch.float32, device).contiguous()

    def forward(self, resid, add, out_dtype, rows=None, out=None):
        return kernels.add_rmsnorm(resid, add, self.weight, self.eps, out_dtype, rows=rows, out=out)
