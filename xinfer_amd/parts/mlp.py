"""Gated feed-forward (SwiGLU): down(silu(gate(x)) * up(x)).

gate and up are concatenated at load into one [2I, H] weight, the product lands in a
packed [T, 2I] buffer and one kernel applies silu(g) * u (reference: MLP::forward,
/root/reference/src/models/layers/mlp.rs:613-633; merge at load mlp.rs:447-466).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import FeedForward, StepContext, register_feed_forward
from .linear import Linear


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        if spec.get("activation", "silu") != "silu":
            raise NotImplementedError(f"activation {spec.get('activation')!r} is not built (silu only)")
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        return [TensorDecl(f"{prefix}.gate_proj.weight", (i, h)),
                TensorDecl(f"{prefix}.up_proj.weight", (i, h)),
                TensorDecl(f"{prefix}.down_proj.weight", (h, i))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        def lin(name):
            t = store.get(name, None, device)
            return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t
        g, u = lin(f"{prefix}.gate_proj.weight"), lin(f"{prefix}.up_proj.weight")
        common = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        self.gate_up = Linear(torch.cat([g.to(common), u.to(common)], dim=0))
        self.down = Linear(lin(f"{prefix}.down_proj.weight"))

    takes_sink = True
    takes_folded = True

    def forward(self, x, ctx: StepContext, sink=None):
        """`x`: rows or a `Folded`; `sink`: see `Part.takes_sink`."""
        m = self.gate_up(x, out_dtype=self.dtype, gated=True)         # gate, up and silu*mul in one pass
        if m is None:
            m = kernels.silu_mul(self.gate_up(x, out_dtype=self.dtype))
        return self.down(m, out_dtype=self.dtype, allow_split=True, sink=sink)   # the next norm adds the parts
