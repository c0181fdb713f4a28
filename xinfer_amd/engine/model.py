"""The architecture-neutral model: embedding, blocks in schedule order, final norm, head.

Built from a `ModelSpec` alone.  The reference's counterpart is Qwen3ForCausalLM
(/root/reference/src/models/qwen3.rs:137-445; forward_inner 311-374): embed, the layer
loop, selection of the wanted rows, final norm, lm_head with float32 logits.  Unlike the
reference, which keeps only the last row of each sequence (qwen3.rs:359-363), any set of
rows may be asked for.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch

from ..config.spec import ModelSpec
from ..parts import (KVNeed, LayerCache, StateNeed, StepContext, Stream, block_class, embedding_class,
                     head_class, norm_class)
from ..weights.store import TensorDecl, WeightStore


@dataclass(frozen=True)
class CacheGroupNeed:
    """Layers whose cache needs are the same kind: all keys (window 0) or a window."""
    window: int
    layers: Tuple[int, ...]             # layer indices that own pages in this group


class CausalLM:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype {dtype} is not supported (float32 or bfloat16)")
        self.spec = spec
        self.dtype = dtype
        self.embedding = embedding_class(spec.embedding.kind)(spec.embedding, dtype)
        self.blocks = [block_class(l.block)(l, dtype) for l in spec.layers]
        self.final_norm = norm_class(spec.final_norm.kind)(spec.final_norm, dtype)
        self.head = head_class(spec.head.kind)(spec.head, dtype)
        for e in spec.schedule:
            if not (0 <= e.layer < len(self.blocks)):
                raise ValueError(f"schedule names layer {e.layer} but the model has {len(self.blocks)}")
            if e.cache_of is not None and not (0 <= e.cache_of < len(self.blocks)):
                raise ValueError(f"schedule entry reads the cache of unknown layer {e.cache_of}")
        self._plan_cache()

    @property
    def graph_safe(self) -> bool:
        """Every part can be recorded into a HIP graph (see `Part.graph_safe`)."""
        return all(p.graph_safe for p in (self.embedding, self.final_norm, self.head, *self.blocks))

    # ---- weights -------------------------------------------------------------
    @classmethod
    def declare(cls, spec: ModelSpec) -> List[TensorDecl]:
        decls = embedding_class(spec.embedding.kind).declare(spec.embedding)
        for l in spec.layers:
            decls += block_class(l.block).declare(l)
        decls += norm_class(spec.final_norm.kind).declare(spec.final_norm, str(spec.final_norm.get("prefix", "")))
        decls += head_class(spec.head.kind).declare(spec.head)
        seen, out = set(), []
        for d in decls:                      # a tied head names the embedding table again
            if d.name not in seen:
                seen.add(d.name)
                out.append(d)
        return out

    def load(self, store: WeightStore, device) -> "CausalLM":
        # tensors of the source that no part asked for are left alone, as the reference leaves them
        self.ignored_tensors = store.check(self.declare(self.spec))
        if self.ignored_tensors:
            shown = ", ".join(self.ignored_tensors[:4]) + (", ..." if len(self.ignored_tensors) > 4 else "")
            print(f"[xinfer_amd] {store.where}: {len(self.ignored_tensors)} tensors the model does not use "
                  f"are ignored ({shown})", file=sys.stderr, flush=True)
        self.device = torch.device(device)
        self.embedding.load(store, "", device)
        for b in self.blocks:
            b.load(store, device)
        self.final_norm.load(store, str(self.spec.final_norm.get("prefix", "")), device)
        self.head.load(store, "", device, shared=self.embedding.table if self.head.tied else None)
        return self

    # ---- cache planning --------------------------------------------------------
    def _plan_cache(self) -> None:
        """Which layers own pages, in which group; which own per-request state."""
        self.kv_needs: Dict[int, KVNeed] = {}
        self.state_needs: Dict[int, StateNeed] = {}
        owners = []
        for e in self.spec.schedule:
            owner = e.layer if e.cache_of is None else e.cache_of
            if owner not in owners:
                owners.append(owner)
        windows: List[int] = []
        by_window: Dict[int, List[int]] = {}
        for l in owners:
            kv = self.blocks[l].cache_need()
            if kv is not None:
                self.kv_needs[l] = kv
                if kv.window not in by_window:
                    by_window[kv.window] = []
                    windows.append(kv.window)
                by_window[kv.window].append(l)
            st = self.blocks[l].state_need()
            if st is not None:
                self.state_needs[l] = st
        self.cache_groups: List[CacheGroupNeed] = [
            CacheGroupNeed(w, tuple(by_window[w])) for w in windows]
        self.group_of_layer: Dict[int, int] = {
            l: g for g, grp in enumerate(self.cache_groups) for l in grp.layers}

    # ---- step ------------------------------------------------------------------
    def forward(self, ids: torch.Tensor, ctx: StepContext, caches: Dict[int, LayerCache],
                want_rows: torch.Tensor) -> torch.Tensor:
        """ids int32 [T]; caches: layer index -> the cache that layer owns; want_rows int32
        [R].  Returns float32 logits [R, vocab]."""
        stream = Stream(self.embedding.forward(ids, ctx), None)
        schedule = self.spec.schedule
        for i, e in enumerate(schedule):
            owner = e.layer if e.cache_of is None else e.cache_of
            c = caches.get(owner)
            if c is None:
                c = LayerCache()
            elif e.cache_of is not None:
                c = LayerCache(c.group, c.pools, c.state, write=False)
            blk = self.blocks[e.layer]
            if getattr(blk, "folds", False):
                # the block that runs next may let this one half do its first norm
                nxt = self.blocks[schedule[i + 1].layer] if i + 1 < len(schedule) else None
                next_norm = nxt.first_norm() if getattr(nxt, "folds", False) else None
                stream = blk.forward(stream, ctx, c, next_norm=next_norm)
            else:
                stream = blk.forward(stream, ctx, c)
        h = self.final_norm.forward(stream.resid, stream.pending, self.dtype, rows=want_rows)
        return self.head.forward(h)
