"""Block arrangements.

"prenorm": x -> norm -> mixer -> (+x, norm) -> feed-forward -> (+r)
(reference: Qwen3DecoderLayer::forward, /root/reference/src/models/qwen3.rs:108-134).
Each residual add is carried out by the norm kernel that follows it: a block hands on
the stream with its feed-forward output still pending, and the next block's first
norm (or the model's final norm) adds it.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.spec import LayerSpec
from ..weights.store import TensorDecl, WeightStore
from .base import (Block, Folded, KVNeed, LayerCache, NormSink, StateNeed, StepContext, Stream,
                   feed_forward_class, mixer_class, norm_class, register_block)

@register_block("prenorm")
class PreNormBlock(Block):
    """Runs two norms: `layer.norms` names the one before the mixer first, then the one before
    the feed-forward.  Every tensor name comes from the `LayerSpec`."""

    def __init__(self, layer: LayerSpec, dtype: torch.dtype):
        super().__init__(layer, dtype)
        self.mixer = mixer_class(layer.mixer.kind)(layer.mixer, dtype)
        self.ffn = feed_forward_class(layer.feed_forward.kind)(layer.feed_forward, dtype)
        (self._name1, n1), (self._name2, n2) = layer.norm_items(2)
        self.norm1 = norm_class(n1.kind)(n1, dtype)
        self.norm2 = norm_class(n2.kind)(n2, dtype)

    @classmethod
    def declare(cls, layer: LayerSpec) -> List[TensorDecl]:
        p = layer.prefix
        out = mixer_class(layer.mixer.kind).declare(layer.mixer, f"{p}.{layer.mixer_name}")
        out += feed_forward_class(layer.feed_forward.kind).declare(layer.feed_forward, f"{p}.{layer.feed_forward_name}")
        for name, n in layer.norm_items(2):
            out += norm_class(n.kind).declare(n, f"{p}.{name}")
        return out

    def load(self, store: WeightStore, device) -> None:
        p = self.layer.prefix
        self.mixer.load(store, f"{p}.{self.layer.mixer_name}", device)
        self.ffn.load(store, f"{p}.{self.layer.feed_forward_name}", device)
        self.norm1.load(store, f"{p}.{self._name1}", device)
        self.norm2.load(store, f"{p}.{self._name2}", device)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.mixer, self.ffn, self.norm1, self.norm2))

    def cache_need(self) -> Optional[KVNeed]:
        return self.mixer.cache_need()

    def state_need(self) -> Optional[StateNeed]:
        return self.mixer.state_need()

    # ---- folding norms into the products around them (parts.base.Folded) ---------------------
    folds = True         # `forward` takes `next_norm` and a stream with `folded`

    def first_norm(self):
        """The norm that a block before this one may half do, or None."""
        return self.norm1 if (self.norm1.foldable and self.mixer.takes_folded) else None

    def forward(self, stream: Stream, ctx: StepContext, cache: LayerCache, next_norm=None) -> Stream:
        """`next_norm`: the first norm of the block that runs next, if that block lets this
        one's feed-forward half do it."""
        if stream.folded is not None:
            if stream.folded.norm is not self.norm1:
                raise RuntimeError("the stream carries a half-done norm of another block")
            h = stream.folded
        else:
            h = self.norm1.forward(stream.resid, stream.pending, self.dtype)
        if self.mixer.takes_sink and self.ffn.takes_folded and self.norm2.foldable:
            a = self.mixer.forward(h, ctx, cache, sink=NormSink(stream.resid, self.norm2))
        else:
            a = self.mixer.forward(h, ctx, cache)
        h2 = a if isinstance(a, Folded) else self.norm2.forward(stream.resid, a, self.dtype)
        if next_norm is not None and self.ffn.takes_sink:
            m = self.ffn.forward(h2, ctx, sink=NormSink(stream.resid, next_norm))
        else:
            m = self.ffn.forward(h2, ctx)
        if isinstance(m, Folded):
            return Stream(stream.resid, None, m)
        return Stream(stream.resid, m)
