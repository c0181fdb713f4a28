"""Token embedding and the language-model head, as kinds of their own registries.

"embedding": x = E[ids] (times `scale` if the spec gives one; Qwen3 gives none) into the
float32 residual stream (reference: /root/reference/src/models/qwen3.rs:211-220,302-309).
"lm_head": logits = h @ W^T in float32; W is the embedding table when the spec says `tied`
(qwen3.rs:267-287,367-373); `softcap` c, if the spec gives one, makes them c * tanh(logits / c).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import Head, StepContext, TokenEmbedding, register_embedding, register_head
from .linear import Linear


@register_embedding("embedding")
class Embedding(TokenEmbedding):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.vocab = int(spec["vocab_size"])
        self.dim = int(spec["dim"])
        self.scale = float(spec.get("scale") or 1.0)
        self.table: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str = "") -> List[TensorDecl]:
        return [TensorDecl(spec["name"], (int(spec["vocab_size"]), int(spec["dim"])))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        t = store.get(self.spec["name"], None, device)
        if self.dtype == torch.float32 or t.dtype != torch.float32:
            t = t.to(self.dtype)
        self.table = t.contiguous()

    def forward(self, ids: torch.Tensor, ctx: Optional[StepContext] = None) -> torch.Tensor:
        return kernels.embed(self.table, ids, scale=self.scale)


@register_head("lm_head")
class LMHead(Head):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.tied = bool(spec.get("tied", False))
        self.softcap = float(spec.get("softcap") or 0.0)
        self.proj: Optional[Linear] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str = "") -> List[TensorDecl]:
        return [TensorDecl(spec["name"], (int(spec["vocab_size"]), int(spec["dim"])))]

    def load(self, store: WeightStore, prefix: str, device, shared: Optional[torch.Tensor] = None) -> None:
        if self.tied and shared is not None:
            self.proj = Linear(shared)
            return
        t = store.get(self.spec["name"], None, device)
        if self.dtype == torch.float32 or t.dtype != torch.float32:
            t = t.to(self.dtype)
        self.proj = Linear(t)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        # float32 logits straight from the float32 sums.  In float32 a row's logits do not depend on
        # how many rows were asked for (one fixed-order kernel); in bfloat16 the kernel is chosen by
        # the number of rows (thin or streaming up to 3, tiled up to 128, the library beyond), each
        # with its own order of sums, so they agree to rounding only
        logits = self.proj(h, out_dtype=torch.float32, skinny_rows=kernels.SKINNY_MAX_ROWS)
        return kernels.softcap_(logits, self.softcap) if self.softcap > 0 else logits
