"""The step function: runs one mixed batch through the model from the cache.

`ModelRunner` owns the model, the device memory of the paged cache (per layer that owns
pages the pools its mixer declares: for attention a K and a V pool,
`[pages, kv_heads, page_size, head_dim]`), the per-request state arenas, and the cache
manager that says which request holds which pages.  A state slot is cleared when the
request it serves runs its first token (a request that starts, or starts again after it
gave way), so a mixer finds zeros there, never another request's state.  `step` takes a list of entries (request, its next tokens, the places whose
logits are wanted), runs exactly those tokens as one batch against what earlier steps
left in the cache, and returns float32 logits for the wanted places.  A decode token is
an entry with one token; prompt portions may be cut anywhere.

The reference's counterpart is ModelRunner::run with prepare_prefill / prepare_decode
(/root/reference/src/core/runner.rs:1018-1217, 1303-1563, 1565-1750), which never mixes
prompt portions and decode tokens in one step and returns one sampled token per
sequence; this one mixes them and leaves sampling to the caller.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import DecodeStepError, BatchArrays, CacheGroup, PagedCacheManager
from ..parts import LayerCache, StepContext
from .model import CausalLM


@dataclass
class StepEntry:
    request: int                       # id of a live request
    tokens: Sequence[int]              # its next tokens (at least one)
    want: Sequence[int] = ()           # indices into `tokens` whose logits are wanted


class StepError(ValueError):
    pass


def _similar(ctx_lens: np.ndarray) -> bool:
    """The sequences of a step are about equally long (kernels may then give each a workgroup of
    its own instead of cutting all into equal pieces)."""
    return bool(ctx_lens.size) and float(ctx_lens.mean()) >= 0.9 * float(ctx_lens.max())


class _Staging:
    """Pinned host buffers through which a step's index arrays reach the device: one copy
    for the 32-bit arrays and one for the 64-bit ones."""

    def __init__(self, device):
        self.device = device
        self._pin = {torch.int32: None, torch.int64: None}
        self._done: Optional[torch.cuda.Event] = None

    def upload(self, parts: Sequence[np.ndarray], dtype: torch.dtype,
               dst: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, List[int]]:
        """Concatenates `parts` into one device tensor (into `dst` if given) and returns it
        with the offset of every part."""
        offsets, n = [], 0
        for p in parts:
            offsets.append(n)
            n += int(p.size)
        pin = self._pin[dtype]
        if pin is None or pin.numel() < n:
            pin = torch.empty((max(1024, 1 << (n - 1).bit_length()),), dtype=dtype, pin_memory=True)
            self._pin[dtype] = pin
        if self._done is not None:
            self._done.synchronize()        # the previous step's copy has left the buffer
        host = pin.numpy()
        for off, p in zip(offsets, parts):
            host[off:off + p.size] = p.reshape(-1)
        if dst is None:
            dst = torch.empty((n,), dtype=dtype, device=self.device)
        elif dst.numel() != n or dst.dtype != dtype:
            raise ValueError("staging: the fixed device buffer does not fit this step's arrays")
        dst.copy_(pin[:n], non_blocking=True)
        return dst, offsets

    def pinned(self, dtype: torch.dtype, n: int) -> np.ndarray:
        """The pinned buffer of `dtype` with room for n elements, free to be written (the copy
        of the step before has left it)."""
        pin = self._pin[dtype]
        if pin is None or pin.numel() < n:
            pin = torch.empty((max(1024, 1 << (n - 1).bit_length()),), dtype=dtype, pin_memory=True)
            self._pin[dtype] = pin
        if self._done is not None:
            self._done.synchronize()
            self._done = None
        return pin.numpy()

    def push(self, dtype: torch.dtype, n: int, dst: torch.Tensor) -> None:
        """Copies the first n elements of the pinned buffer into `dst`."""
        if dst.numel() != n or dst.dtype != dtype:
            raise ValueError("staging: the fixed device buffer does not fit this step's arrays")
        dst.copy_(self._pin[dtype][:n], non_blocking=True)

    def mark(self) -> None:
        self._done = torch.cuda.Event()
        self._done.record()


@dataclass
class _DecodeGraph:
    graph: Any
    dev32: torch.Tensor
    dev64: torch.Tensor
    logits: torch.Tensor            # [B, vocab], rewritten by every replay
    want: torch.Tensor              # int32 [B]: this step's wanted rows (first R valid)
    keep: Tuple[Any, ...] = ()      # everything else the recorded kernels read: it must stay
                                    # allocated for as long as the graph may be replayed

    @property
    def nbytes(self) -> int:
        """What the graph holds for itself between replays: its logits and its index arrays."""
        return sum(t.numel() * t.element_size() for t in (self.dev32, self.dev64, self.logits))


def context_bucket(longest: int) -> int:
    """The longest context a recorded decode step is laid out for, given the step's longest: the
    next multiple of 1,024 up to 16,384, of an eighth of the power of two below beyond that (eight
    buckets an octave).  Kernels whose grid depends on the longest context are recorded for the
    bucket's upper bound; with buckets an eighth apart or closer what they plan for is near what
    they get (powers of two planned the attention's workgroups for up to twice the keys)."""
    longest = max(1, int(longest))
    if longest <= 16384:
        return -(-longest // 1024) * 1024
    step = 1 << (longest.bit_length() - 1 - 3)
    return -(-longest // step) * step


GRAPHS_MOST = 48                    # recorded decode graphs kept at a time, and
GRAPH_BYTES_MOST = 1 << 30          # the bytes they may hold together; the least recently used goes first


class ModelRunner:
    def __init__(self, model: CausalLM, page_size: int, num_pages, max_requests: int,
                 use_graphs: bool = True, graph_max_batch: Optional[int] = None, graph_after: Optional[int] = None,
                 graphs_most: int = GRAPHS_MOST, graph_bytes_most: int = GRAPH_BYTES_MOST):
        """`num_pages`: pages of every group's pool, or a list with one count per group.
        `use_graphs`: record decode steps of up to `graph_max_batch` requests as HIP graphs; a
        (batch size, context bucket) is recorded the `graph_after`-th time it is seen, so that
        batch sizes that merely pass by (requests finishing one after the other) do not pay
        for a recording.  The step that records runs its tokens once, launch by launch, and then
        captures the same launches without running them: a recording costs two passes of the host
        over the model and the graph's instantiation (12 to 25 ms at 8B to 32B sizes on an MI355X); a replay saves what
        the host's launches of a step take beyond the kernels' own time: everything for a small
        model, 0.1 to 0.2 ms a step for a large one, whose kernels outlast the launches.  Left to
        the runner, the count is 3 for a model whose step is bound by the host and 12 otherwise,
        and `graph_max_batch` 256 for such a model (its launches cost more than its kernels at
        any batch size) and 64 otherwise.  At most `graphs_most` graphs holding `graph_bytes_most`
        bytes (their logits, 39 MB at 64 rows of 151,936, and index arrays) are kept; beyond that
        the least recently replayed one is dropped and its key starts counting sightings again
        (the reference records batch sizes 1 to 32 once, /root/reference/src/utils/graph.rs:415-420)."""
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
            pools = {}
            for pool in kv.pools:         # what the mixer declares, page by page
                if pool.name in pools or sum(1 for s in pool.shape if s < 0) != 1:
                    raise ValueError(f"layer {layer}: pool {pool.name!r} of shape {pool.shape} must have a name of its "
                                     "own and exactly one axis of the page's length")
                by = -min(pool.shape)      # PAGE: 1; PAGE_BY_8: 8
                if self.page_size % by:
                    raise ValueError(f"layer {layer}: pool {pool.name!r} keeps its pages in groups of {by} tokens: "
                                     f"the page size {self.page_size} must be a multiple of {by}")
                shape = (groups[g].num_pages, *(self.page_size // by if s < 0 else int(s) for s in pool.shape))
                pools[pool.name] = torch.zeros(shape, dtype=pool.dtype or model.dtype, device=self.device)
            self.layer_caches[layer] = LayerCache(group=g, pools=pools)
        self._state_arenas: List[torch.Tensor] = []
        for layer, st in model.state_needs.items():
            arena = torch.zeros((self.max_requests, *st.shape), dtype=st.dtype, device=self.device)
            self._state_arenas.append(arena)
            if layer in self.layer_caches:
                self.layer_caches[layer].state = arena
            else:
                self.layer_caches[layer] = LayerCache(state=arena)
        self._empty_f32 = torch.empty((1, 0), dtype=torch.float32, device=self.device)
        self._staging = _Staging(self.device)
        self.use_graphs = bool(use_graphs) and model.graph_safe
        # a step's kernels take about weights / 4 TB/s, its launches about 100 us a layer
        size = 2 if model.dtype == torch.bfloat16 else 4
        weights = size * sum(int(np.prod(d.shape)) for d in type(model).declare(model.spec))
        host_bound = weights / 4e12 < 0.5 * max(1, len(model.spec.layers)) * 100e-6
        if graph_after is None:
            graph_after = 3 if host_bound else 12
        if graph_max_batch is None:
            graph_max_batch = 256 if host_bound else 64
        self.graph_after = max(1, int(graph_after))
        self.graph_max_batch = int(graph_max_batch)
        self._graphs: Dict[Tuple[int, int, bool], _DecodeGraph] = {}     # in order of last use, oldest first
        self.graphs_most = max(1, int(graphs_most))
        self.graph_bytes_most = int(graph_bytes_most)
        self.graphs_dropped = 0
        self._seen: Dict[Tuple[int, int, bool], int] = {}
        self._graph_pool = None
        self._device_tokens = None          # the step's tokens that live on the device (see `step`)
        self._tok_pin: Optional[torch.Tensor] = None
        self._tok_pin_free = None
        # widest block table a request can have: the fixed width of a recorded step's tables
        self._max_table = max(1, -(-model.spec.max_positions // self.page_size))
        self.graph_replays = 0

    # ---- requests ---------------------------------------------------------------
    def add_request(self, rid: int) -> int:
        """Makes a request live; returns its state slot."""
        return self.cache.add_request(rid)

    def release(self, rid: int) -> int:
        """Gives back everything the request holds; returns the number of pages."""
        return self.cache.release(rid)

    def length(self, rid: int) -> int:
        return self.cache.length(rid)

    def _clear_state(self, slots: Sequence[int]) -> None:
        """Zeroes the given state slots in every arena (a slot keeps what the request before left)."""
        idx = torch.tensor([int(s) for s in slots], dtype=torch.int64, device=self.device)
        for arena in self._state_arenas:
            arena.index_fill_(0, idx, 0)

    # ---- the step -----------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], reserved: bool = False,
             device_tokens: Optional[Tuple[torch.Tensor, Sequence[int], Sequence[int]]] = None) -> torch.Tensor:
        """Runs the entries' tokens as one batch.  Returns float32 [wanted, vocab] in the
        order of the entries and of each entry's `want`.  With `reserved` the caller (the
        scheduler) has reserved the pages already and also records afterwards that the
        tokens are in the cache; without it this call does both.
        `device_tokens` = (ids, places, rows): tokens that are not known on the host yet.  The
        token at place `places[i]` of the step's tokens (counted over all entries, in order) is
        `ids[rows[i]]`, an int32 tensor on the device that an earlier step's sampling wrote (the
        entries hold any valid id there); it is put in place on the device, in stream order, and
        nothing waits for it."""
        self._device_tokens = device_tokens
        try:
            return self._step(entries, reserved)
        finally:
            self._device_tokens = None

    def _put_device_tokens(self, ids: torch.Tensor) -> None:
        """Overwrites the places of `ids` (the step's token ids on the device) that `step` was
        given device tokens for."""
        if self._device_tokens is None:
            return
        src, places, rows = self._device_tokens
        n = len(places)
        if n == 0:
            return
        if max(places) >= ids.numel() or max(rows) >= src.numel() or min(places) < 0 or min(rows) < 0:
            raise StepError("a device token's place or row is outside the step")
        if n == ids.numel() == src.numel() and list(places) == list(rows) == list(range(n)):
            ids.copy_(src)               # every token, in order: the usual step of decoding requests
            return
        # the two index arrays go up through pinned memory (a copy from ordinary memory would wait for the GPU)
        if self._tok_pin is None or self._tok_pin.numel() < 2 * n:
            self._tok_pin = torch.empty((max(1024, 2 * n),), dtype=torch.int64, pin_memory=True)
        if self._tok_pin_free is not None:
            self._tok_pin_free.synchronize()
        host = self._tok_pin[:2 * n].view(2, n)
        host.copy_(torch.tensor([list(places), list(rows)], dtype=torch.int64))
        idx = torch.empty((2, n), dtype=torch.int64, device=self.device)
        idx.copy_(host, non_blocking=True)
        self._tok_pin_free = torch.cuda.Event()
        self._tok_pin_free.record()
        ids.index_copy_(0, idx[0], src.index_select(0, idx[1]))

    def _step(self, entries: Sequence[StepEntry], reserved: bool) -> torch.Tensor:
        spec = self.model.spec
        if not entries:
            return torch.empty((0, spec.vocab_size), dtype=torch.float32, device=self.device)
        B = len(entries)
        single = all(len(e.tokens) == 1 for e in entries)
        if single and self.use_graphs and B <= self.graph_max_batch and self._graphs:
            if self._state_arenas:       # a request whose first token this is gets a clean slot
                ids_ = np.fromiter((e.request for e in entries), np.int64, B)
                fresh = self.cache.lengths(ids_) == 0
                if fresh.any():
                    self._clear_state([self.cache.state_slot(int(r)) for r in ids_[fresh]])
            logits = self._decode_recorded(entries, reserved)
            if logits is not None:
                return logits
        if single:
            # a step of single tokens (the hot path of decoding): checked and reserved in a few
            # calls for all entries together
            rid_arr = np.fromiter((e.request for e in entries), np.int64, B)
            counts_arr = np.ones(B, np.int32)
            ids_host = np.fromiter((e.tokens[0] for e in entries), np.int64, B)
            if len(set(rid_arr.tolist())) != B:
                raise StepError("a request appears twice in one step")
            lengths = self.cache.lengths(rid_arr)
            if lengths.min() < 0:
                raise StepError(f"request {int(rid_arr[int(lengths.argmin())])} is not live")
            if lengths.max() + 1 > spec.max_positions:
                b = int(lengths.argmax())
                raise StepError(f"request {int(rid_arr[b])}: {int(lengths[b]) + 1} tokens exceed the "
                                f"model's {spec.max_positions} positions")
            rows = []
            for b, e in enumerate(entries):
                for w in e.want:
                    if w != 0:
                        raise StepError(f"request {e.request}: wanted place {w} is outside its 1 tokens")
                    rows.append(b)
        else:
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
            rid_arr = np.asarray(rids, dtype=np.int64)
            counts_arr = np.asarray(counts, dtype=np.int32)
            ids_host = np.asarray(all_tokens, dtype=np.int64)
        if ids_host.min() < 0 or ids_host.max() >= spec.vocab_size:
            raise StepError(f"a token id is outside the vocabulary of {spec.vocab_size}")
        if not reserved:
            self.cache.reserve_many(rid_arr, counts_arr)   # OutOfPages leaves every request's length as it was
        decode = self.use_graphs and int(counts_arr.max()) == 1 and B <= self.graph_max_batch
        arrays = self.cache.build_batch(rid_arr, counts_arr, max_pages=self._max_table if decode else None)
        if self._state_arenas:           # requests that run their first token get a clean slot
            fresh = (arrays.ctx_lens - np.diff(arrays.cu_q)) == 0
            if fresh.any():
                self._clear_state(arrays.state_slots[fresh].tolist())
        ids32 = ids_host.astype(np.int32)
        rows32 = np.asarray(rows, dtype=np.int32)
        if decode:
            logits = self._replay_decode(arrays, ids32, rows32)
        else:
            ctx, ids, want_rows, _, _ = self._context(arrays, ids32, rows32)
            self._put_device_tokens(ids)
            logits = self.model.forward(ids, ctx, self.layer_caches, want_rows)
        if not reserved:
            self.cache.commit_many(rid_arr, counts_arr)
        return logits

    def _decode_recorded(self, entries: Sequence[StepEntry], reserved: bool) -> Optional[torch.Tensor]:
        """A step of single tokens whose graph is recorded already: one call into the cache
        manager checks the requests, reserves their pages and writes the step's arrays straight
        into the pinned buffers; two copies and a replay follow.  Returns None (nothing done
        but, possibly, the reservation, which the general path repeats harmlessly) if the step
        has no recorded graph yet."""
        spec = self.model.spec
        B = len(entries)
        G = len(self.cache.groups)
        P = self._max_table
        rid_arr = np.fromiter((e.request for e in entries), np.int64, B)
        tokens = np.fromiter((e.tokens[0] for e in entries), np.int32, B)
        rows = np.fromiter((b for b, e in enumerate(entries) for _ in e.want), np.int32)
        if any(w != 0 for e in entries for w in e.want):
            raise StepError("a wanted place is outside an entry's 1 tokens")
        n32, n64 = 6 * B + 1 + G * B * P, (2 + G) * B
        host32 = self._staging.pinned(torch.int32, n32)
        host64 = self._staging.pinned(torch.int64, n64)
        try:
            longest, similar = self.cache.decode_step(rid_arr, tokens, not reserved, spec.vocab_size,
                                                      spec.max_positions, P, rows, host32, host64)
        except DecodeStepError as ex:
            rid = int(rid_arr[ex.entry]) if 0 <= ex.entry < B else -1
            raise StepError({-1: f"request {rid} is not live", -2: f"request {rid} appears twice in one step",
                             -3: f"request {rid}: its tokens exceed the model's {spec.max_positions} positions",
                             -4: f"a token id is outside the vocabulary of {spec.vocab_size}"}.get(
                                 ex.kind, f"the step could not be prepared ({ex.kind})")) from None
        bucket = context_bucket(longest)
        g = self._graphs.get((B, bucket, similar))
        if g is None:
            return None
        self._used(g, (B, bucket, similar))
        self._staging.push(torch.int32, n32, g.dev32)
        self._staging.push(torch.int64, n64, g.dev64)
        self._staging.mark()
        self._put_device_tokens(g.dev32[:B])        # the token ids lead the 32-bit arrays
        g.graph.replay()
        self.graph_replays += 1
        if not reserved:
            self.cache.commit_many(rid_arr, np.ones(B, np.int32))
        if rows.size == B and np.array_equal(rows, np.arange(B)):
            return g.logits.clone()
        return g.logits.index_select(0, g.want[:rows.size])

    # ---- index arrays on the device -------------------------------------------------
    def _context(self, a: BatchArrays, ids32: np.ndarray, rows32: np.ndarray, dst32=None, dst64=None,
                 max_ctx_len: Optional[int] = None, host_lengths: bool = True):
        """Uploads the step's arrays (two copies) and returns (StepContext, ids, wanted rows,
        32-bit buffer, 64-bit buffer); the first three are views of the two buffers."""
        dev = self.device
        G = len(self.cache.groups)
        T, B = a.num_tokens, a.num_seqs
        d32, o32, d64, o64 = self._upload(a, ids32, rows32, dst32, dst64)
        v32 = lambda i, n: d32[o32[i]:o32[i] + n]
        P = a.max_pages
        tables = v32(6, G * B * P).view(G, B, P)
        slots = d64[o64[1]:o64[1] + G * T].view(G, T)
        q_lens = np.diff(a.cu_q)
        ctx = StepContext(
            num_tokens=T, num_seqs=B, dtype=self.model.dtype, device=dev,
            positions=v32(1, T), tok_seq=v32(2, T), cu_q=v32(3, B + 1), ctx_lens=v32(4, B),
            state_slots=d64[o64[0]:o64[0] + B],
            slots=[slots[g] for g in range(G)], block_tables=[tables[g] for g in range(G)],
            cu_q_host=a.cu_q.tolist() if host_lengths else (),
            ctx_lens_host=a.ctx_lens.tolist() if host_lengths else (),
            max_q_len=int(q_lens.max()),
            max_ctx_len=int(a.ctx_lens.max()) if max_ctx_len is None else int(max_ctx_len),
            similar_lengths=_similar(a.ctx_lens),
            no_slots=d64[o64[2]:o64[2] + T], empty_f32=self._empty_f32)
        return ctx, v32(0, T), v32(5, rows32.size), d32, d64

    def _upload(self, a: BatchArrays, ids32: np.ndarray, rows32: np.ndarray, dst32=None, dst64=None):
        """The step's arrays to the device in two copies (into the fixed buffers of a recorded
        step if given); returns both buffers with the offsets of their parts."""
        no_slots = np.full(a.num_tokens, -1, dtype=np.int64)
        parts32 = [ids32, a.positions, a.tok_seq, a.cu_q, a.ctx_lens, rows32, a.block_tables]
        parts64 = [a.state_slots.astype(np.int64), a.slots, no_slots]
        d32, o32 = self._staging.upload(parts32, torch.int32, dst32)
        d64, o64 = self._staging.upload(parts64, torch.int64, dst64)
        self._staging.mark()
        return d32, o32, d64, o64

    # ---- decode steps as HIP graphs ---------------------------------------------------
    def _used(self, g: _DecodeGraph, key) -> None:
        """Moves a graph to the young end of the order of last use."""
        if next(reversed(self._graphs)) != key:
            del self._graphs[key]
            self._graphs[key] = g

    def _drop_least_used(self, keep) -> None:
        """Drops the least recently used graphs until count and bytes are within their bounds (the
        one just recorded stays).  A dropped graph's memory goes back to the graphs' pool once its
        last replay has finished."""
        while len(self._graphs) > 1 and (len(self._graphs) > self.graphs_most
                                         or sum(g.nbytes for g in self._graphs.values()) > self.graph_bytes_most):
            key = next(k for k in self._graphs if k != keep)
            torch.cuda.current_stream(self.device).synchronize()
            del self._graphs[key]
            self._seen.pop(key, None)
            self.graphs_dropped += 1

    def _replay_decode(self, a: BatchArrays, ids32: np.ndarray, rows32: np.ndarray) -> torch.Tensor:
        """A step of single tokens.  The graph of (batch size, context bucket) computes the
        logits of every row; the wanted rows are gathered afterwards.  Kernels whose grid
        depends on the longest context are recorded for the bucket's upper bound (work
        beyond a request's own length ends at once)."""
        B = a.num_seqs
        longest = int(a.ctx_lens.max())
        bucket = context_bucket(longest)
        key = (B, bucket, _similar(a.ctx_lens))     # what kernels choose their shapes from
        all_rows = np.zeros(B, dtype=np.int32)
        all_rows[:rows32.size] = rows32
        g = self._graphs.get(key)
        if g is None:
            self._seen[key] = self._seen.get(key, 0) + 1
            if self._seen[key] < self.graph_after:         # not yet: launch by launch
                ctx, ids, want_rows, _, _ = self._context(a, ids32, rows32)
                self._put_device_tokens(ids)
                return self.model.forward(ids, ctx, self.layer_caches, want_rows)
            ctx, ids, want, d32, d64 = self._context(a, ids32, all_rows, max_ctx_len=bucket, host_lengths=False)
            self._put_device_tokens(ids)
            every_row = torch.arange(B, dtype=torch.int32, device=self.device)
            cur = torch.cuda.current_stream(self.device)
            side = torch.cuda.Stream(self.device)
            side.wait_stream(cur)
            with torch.cuda.stream(side):       # this step's own run; it also warms every kernel up
                logits = self.model.forward(ids, ctx, self.layer_caches, every_row)
            cur.wait_stream(side)
            logits.record_stream(cur)           # allocated on the side stream, read on this one from here on
            torch.cuda.synchronize(self.device)
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                recorded = self.model.forward(ids, ctx, self.layer_caches, every_row)
            g = _DecodeGraph(graph, d32, d64, recorded, want, keep=(every_row, ctx, ids))
            self._graphs[key] = g
            self._drop_least_used(keep=key)
            # the step has run once, above; the capture ran nothing and the graph is first replayed
            # by the next step of this key.  A part that updates per-request state in place is
            # thus advanced once a step, also in the step that records.
            if rows32.size == B and np.array_equal(rows32, np.arange(B)):
                return logits
            return logits.index_select(0, want[:rows32.size])
        else:
            self._used(g, key)
            self._upload(a, ids32, all_rows, g.dev32, g.dev64)
            self._put_device_tokens(g.dev32[:B])
        g.graph.replay()
        self.graph_replays += 1
        if rows32.size == B and np.array_equal(rows32, np.arange(B)):
            return g.logits.clone()
        return g.logits.index_select(0, g.want[:rows32.size])
