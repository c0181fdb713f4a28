"""The step function: runs one mixed batch through the model from the cache.

`ModelRunner` owns the model, the device memory of the paged cache (one K and one V
pool per layer that owns pages, `[pages, kv_heads, page_size, head_dim]`), the
per-request state arenas, and the cache manager that says which request holds which
pages.  `step` takes a list of entries (request, its next tokens, the places whose
logits are wanted), runs exactly those tokens as one batch against what earlier steps
left in the cache, and returns float32 logits for the wanted places.  A decode token is
an entry with one token; prompt portions may be cut anywhere.

The reference's counterpart is ModelRunner::run with prepare_prefill / prepare_decode
(/root/reference/src/core/runner.rs:1018-1217, 1303-1563, 1565-1750), which never mixes
prompt portions and decode tokens in one step and returns one sampled token per
sequence; this one mixes them and leaves sampling to the caller.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import BatchArrays, CacheGroup, OutOfPages, PagedCacheManager
from ..parts import LayerCache, StepContext
from .model import CausalLM


@dataclass
class StepEntry:
    request: int                       # id of a live request
    tokens: Sequence[int]              # its next tokens (at least one)
    want: Sequence[int] = ()           # indices into `tokens` whose logits are wanted


class StepError(ValueError):
    pass


class ModelRunner:
    def __init__(self, model: CausalLM, page_size: int, num_pages, max_requests: int):
        """`num_pages`: pages of every group's pool, or a list with one count per group."""
        if not torch.cuda.is_available():
            raise RuntimeError("xinfer_amd runs on an AMD GPU only: no HIP device is visible")
        self.model = model
        self.device = model.device
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        needs = model.cache_groups
        if isinstance(num_pages, int):
            num_pages = [num_pages] * max(1, len(needs))
        if len(num_pages) != max(1, len(needs)):
            raise ValueError(f"{len(num_pages)} page counts for {len(needs)} cache groups")
        groups = [CacheGroup(self.page_size, int(n), g.window) for g, n in zip(needs, num_pages)]
        if not groups:                  # a model without paged layers still has state slots
            groups = [CacheGroup(self.page_size, 0, 0)]
        self.cache = PagedCacheManager(groups, self.max_requests)
        self.layer_caches: Dict[int, LayerCache] = {}
        for layer, kv in model.kv_needs.items():
            g = model.group_of_layer[layer]
            shape = (groups[g].num_pages, kv.num_kv_heads, self.page_size, kv.head_dim)
            v_shape = (shape[0], shape[1], shape[3], shape[2]) if kv.v_transposed else shape
            self.layer_caches[layer] = LayerCache(
                group=g,
                k=torch.zeros(shape, dtype=model.dtype, device=self.device),
                v=torch.zeros(v_shape, dtype=model.dtype, device=self.device))
        for layer, st in model.state_needs.items():
            arena = torch.zeros((self.max_requests, *st.shape), dtype=st.dtype, device=self.device)
            if layer in self.layer_caches:
                self.layer_caches[layer].state = arena
            else:
                self.layer_caches[layer] = LayerCache(state=arena)
        self._empty_f32 = torch.empty((1, 0), dtype=torch.float32, device=self.device)

    # ---- requests ---------------------------------------------------------------
    def add_request(self, rid: int) -> int:
        """Makes a request live; returns its state slot."""
        return self.cache.add_request(rid)

    def release(self, rid: int) -> int:
        """Gives back everything the request holds; returns the number of pages."""
        return self.cache.release(rid)

    def length(self, rid: int) -> int:
        return self.cache.length(rid)

    # ---- the step -----------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], reserved: bool = False) -> torch.Tensor:
        """Runs the entries' tokens as one batch.  Returns float32 [wanted, vocab] in the
        order of the entries and of each entry's `want`.  With `reserved` the caller (the
        scheduler) has reserved the pages already and also records afterwards that the
        tokens are in the cache; without it this call does both."""
        spec = self.model.spec
        if not entries:
            return torch.empty((0, spec.vocab_size), dtype=torch.float32, device=self.device)
        seen = set()
        rids, counts, all_tokens, rows = [], [], [], []
        base = 0
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request}: an entry needs at least one token")
            if e.request in seen:
                raise StepError(f"request {e.request} appears twice in one step")
            seen.add(e.request)
            if not self.cache.has(e.request):
                raise StepError(f"request {e.request} is not live")
            if self.cache.length(e.request) + n > spec.max_positions:
                raise StepError(
                    f"request {e.request}: {self.cache.length(e.request) + n} tokens exceed the "
                    f"model's {spec.max_positions} positions")
            for w in e.want:
                if not (0 <= w < n):
                    raise StepError(f"request {e.request}: wanted place {w} is outside its {n} tokens")
                rows.append(base + int(w))
            rids.append(e.request)
            counts.append(n)
            all_tokens.extend(int(t) for t in e.tokens)
            base += n
        ids_host = np.asarray(all_tokens, dtype=np.int64)
        if ids_host.min() < 0 or ids_host.max() >= spec.vocab_size:
            raise StepError(f"a token id is outside the vocabulary of {spec.vocab_size}")
        if not reserved:
            for rid, n in zip(rids, counts):
                self.cache.reserve(rid, n)      # OutOfPages leaves every request's length as it was
        arrays = self.cache.build_batch(rids, counts)
        ctx = self._context(arrays)
        ids = torch.from_numpy(ids_host.astype(np.int32)).to(self.device)
        want_rows = torch.tensor(rows, dtype=torch.int32, device=self.device)
        logits = self.model.forward(ids, ctx, self.layer_caches, want_rows)
        if not reserved:
            for rid, n in zip(rids, counts):
                self.cache.commit(rid, n)
        return logits

    def _context(self, a: BatchArrays) -> StepContext:
        dev = self.device
        to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
        G = len(self.cache.groups)
        q_lens = np.diff(a.cu_q)
        return StepContext(
            num_tokens=a.num_tokens, num_seqs=a.num_seqs, dtype=self.model.dtype, device=dev,
            positions=to(a.positions), tok_seq=to(a.tok_seq), cu_q=to(a.cu_q),
            ctx_lens=to(a.ctx_lens), state_slots=to(a.state_slots.astype(np.int64)),
            slots=[to(a.slots[g]) for g in range(G)],
            block_tables=[to(a.block_tables[g]) for g in range(G)],
            cu_q_host=a.cu_q.tolist(), ctx_lens_host=a.ctx_lens.tolist(),
            max_q_len=int(q_lens.max()), max_ctx_len=int(a.ctx_lens.max()),
            no_slots=torch.full((a.num_tokens,), -1, dtype=torch.int64, device=dev),
            empty_f32=self._empty_f32)
