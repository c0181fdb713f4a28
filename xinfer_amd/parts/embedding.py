"""Token embedding and the language-model head.

Embedding: x = E[ids], no scaling, into the float32 residual stream (reference:
/root/reference/src/models/qwen3.rs:211-220,302-309).  Head: logits = h @ W^T in float32
output; W is the embedding table when the model ties them (qwen3.rs:267-287,367-373).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import Part
from .linear import Linear


class Embedding(Part):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.vocab = int(spec["vocab_size"])
        self.dim = int(spec["dim"])
        self.table: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str = "") -> List[TensorDecl]:
        return [TensorDecl(spec["name"], (int(spec["vocab_size"]), int(spec["dim"])))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        t = store.get(self.spec["name"], None, device)
        if self.dtype == torch.float32 or t.dtype != torch.float32:
            t = t.to(self.dtype)
        self.table = t.contiguous()

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return kernels.embed(self.table, ids)


class LMHead(Part):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.tied = bool(spec.get("tied", False))
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
        # float32 logits straight from the float32 sums for any number of rows; the streaming
        # kernel serves every decode batch here, so a row's logits do not depend on how many
        # rows were asked for
        return self.proj(h, out_dtype=torch.float32, skinny_rows=kernels.SKINNY_MAX_ROWS)
