"""Python face of the native cache manager (csrc/host/cache.{h,cpp}).

`CacheGroup` describes one group of layers with the same needs; `PagedCacheManager`
owns the page pools' bookkeeping, the block table of every live request per group and
the per-request state slots.  It holds no device memory: the model allocates the pools
(`[pages, kv_heads, page_size, head_dim]` per layer) from the group descriptions.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from ..csrc.build import load_host


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A pool has too few free pages for what was asked; nothing was changed."""


@dataclass(frozen=True)
class CacheGroup:
    page_size: int
    num_pages: int
    window: int = 0          # 0: every key is kept; w > 0: only the last w keys are needed


_I32P = ctypes.POINTER(ctypes.c_int32)
_I64P = ctypes.POINTER(ctypes.c_int64)


def _bind(lib):
    if getattr(lib, "_xi_cm_bound", False):
        return lib
    vp, i, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    sig = {
        "xi_cm_create": (vp, [i, _I32P, _I32P, _I32P, i]),
        "xi_cm_destroy": (None, [vp]),
        "xi_cm_num_groups": (i, [vp]),
        "xi_cm_free_pages": (i, [vp, i]),
        "xi_cm_free_state_slots": (i, [vp]),
        "xi_cm_live_requests": (i, [vp]),
        "xi_cm_has": (i, [vp, i64]),
        "xi_cm_add_request": (i, [vp, i64]),
        "xi_cm_pages_needed": (i, [vp, i64, i64, i]),
        "xi_cm_can_reserve": (i, [vp, i64, i64]),
        "xi_cm_reserve": (i, [vp, i64, i64]),
        "xi_cm_commit": (i, [vp, i64, i64]),
        "xi_cm_release": (i, [vp, i64]),
        "xi_cm_length": (i64, [vp, i64]),
        "xi_cm_state_slot": (i, [vp, i64]),
        "xi_cm_block_table": (i, [vp, i64, i, _I32P, i]),
        "xi_cm_check": (i, [vp, ctypes.c_char_p, i]),
        "xi_cm_last_error": (ctypes.c_char_p, [vp]),
        "xi_cm_max_table_len": (i, [vp, i, _I64P]),
        "xi_cm_lengths": (None, [vp, i, _I64P, _I64P]),
        "xi_cm_decode_step": (i, [vp, i, _I64P, _I32P, i, i, i64, i, _I32P, i, _I32P, _I64P, _I32P, _I32P]),
        "xi_cm_reserve_many": (i, [vp, i, _I64P, _I32P]),
        "xi_cm_commit_many": (i, [vp, i, _I64P, _I32P]),
        "xi_cm_build_batch": (i, [vp, i, _I64P, _I32P, _I32P, _I32P, _I32P, _I32P, _I32P,
                                  _I64P, _I32P, i, i]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._xi_cm_bound = True
    return lib


@dataclass
class BatchArrays:
    """Host arrays of one step, in the layout the kernels read."""
    num_tokens: int
    num_seqs: int
    max_pages: int
    positions: np.ndarray      # [T] int32
    tok_seq: np.ndarray        # [T] int32
    cu_q: np.ndarray           # [B+1] int32
    ctx_lens: np.ndarray       # [B] int32
    state_slots: np.ndarray    # [B] int32
    slots: np.ndarray          # [G, T] int64
    block_tables: np.ndarray   # [G, B, max_pages] int32


class DecodeStepError(Exception):
    """`decode_step` refused entry `entry`: kind -1 not live, -2 twice, -3 past the model's
    positions, -4 token outside the vocabulary, -6 a wanted row outside the step, -7 no batch."""

    def __init__(self, kind: int, entry: int):
        super().__init__(f"decode step: kind {kind}, entry {entry}")
        self.kind, self.entry = kind, entry


class PagedCacheManager:
    def __init__(self, groups: Sequence[CacheGroup], max_requests: int):
        if not groups:
            raise CacheError("a cache manager needs at least one group")
        self._lib = _bind(load_host())
        self.groups: List[CacheGroup] = list(groups)
        self.max_requests = int(max_requests)
        ps = (ctypes.c_int32 * len(groups))(*[g.page_size for g in groups])
        npg = (ctypes.c_int32 * len(groups))(*[g.num_pages for g in groups])
        win = (ctypes.c_int32 * len(groups))(*[g.window for g in groups])
        self._h = self._lib.xi_cm_create(len(groups), ps, npg, win, self.max_requests)
        if not self._h:
            raise CacheError(f"bad cache groups {groups!r} or max_requests {max_requests}")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.xi_cm_destroy(h)

    # ---- queries ------------------------------------------------------------
    def free_pages(self, group: int = 0) -> int:
        return self._lib.xi_cm_free_pages(self._h, group)

    def free_state_slots(self) -> int:
        return self._lib.xi_cm_free_state_slots(self._h)

    def live_requests(self) -> int:
        return self._lib.xi_cm_live_requests(self._h)

    def has(self, rid: int) -> bool:
        return bool(self._lib.xi_cm_has(self._h, rid))

    def length(self, rid: int) -> int:
        n = self._lib.xi_cm_length(self._h, rid)
        if n < 0:
            raise CacheError(f"unknown request {rid}")
        return n

    def state_slot(self, rid: int) -> int:
        return self._lib.xi_cm_state_slot(self._h, rid)

    def block_table(self, rid: int, group: int = 0) -> List[int]:
        cap = 1 << 16
        buf = (ctypes.c_int32 * cap)()
        n = self._lib.xi_cm_block_table(self._h, rid, group, buf, cap)
        if n < 0:
            raise CacheError(f"unknown request {rid} or group {group}")
        return list(buf[:min(n, cap)])

    def pages_needed(self, rid: int, n: int, group: int = 0) -> int:
        return self._lib.xi_cm_pages_needed(self._h, rid, n, group)

    def can_reserve(self, rid: int, n: int) -> bool:
        return bool(self._lib.xi_cm_can_reserve(self._h, rid, n))

    def check(self) -> None:
        buf = ctypes.create_string_buffer(256)
        if not self._lib.xi_cm_check(self._h, buf, 256):
            raise CacheError(f"cache bookkeeping is inconsistent: {buf.value.decode()}")

    # ---- changes ------------------------------------------------------------
    def add_request(self, rid: int) -> int:
        s = self._lib.xi_cm_add_request(self._h, rid)
        if s == -2:
            raise CacheError(f"request {rid} is live already")
        if s < 0:
            raise CacheError(f"no free state slot for request {rid} "
                             f"({self.max_requests} requests may be live at a time)")
        return s

    def reserve(self, rid: int, n: int) -> None:
        if not self._lib.xi_cm_reserve(self._h, rid, n):
            msg = self._lib.xi_cm_last_error(self._h).decode()
            if not self.has(rid):
                raise CacheError(msg)
            raise OutOfPages(f"request {rid} needs pages for {n} more tokens: {msg}")

    def commit(self, rid: int, n: int) -> int:
        r = self._lib.xi_cm_commit(self._h, rid, n)
        if r < 0:
            raise CacheError(self._lib.xi_cm_last_error(self._h).decode())
        return r

    # ---- a step's worth in one call ------------------------------------------
    def lengths(self, rids: np.ndarray) -> np.ndarray:
        """Cached lengths of the requests `rids` (int64 array); -1 where a request is not live."""
        out = np.empty(rids.size, np.int64)
        self._lib.xi_cm_lengths(self._h, int(rids.size), rids.ctypes.data_as(_I64P), out.ctypes.data_as(_I64P))
        return out

    def reserve_many(self, rids: np.ndarray, counts: np.ndarray) -> None:
        """`reserve` for every request in turn (rids int64, counts int32); the first that
        cannot be served raises as `reserve` does, the ones before it keep their pages."""
        b = self._lib.xi_cm_reserve_many(self._h, int(rids.size), rids.ctypes.data_as(_I64P),
                                         counts.ctypes.data_as(_I32P))
        if b >= 0:
            msg = self._lib.xi_cm_last_error(self._h).decode()
            if not self.has(int(rids[b])):
                raise CacheError(msg)
            raise OutOfPages(f"request {int(rids[b])} needs pages for {int(counts[b])} more tokens: {msg}")

    def commit_many(self, rids: np.ndarray, counts: np.ndarray) -> None:
        if self._lib.xi_cm_commit_many(self._h, int(rids.size), rids.ctypes.data_as(_I64P),
                                       counts.ctypes.data_as(_I32P)) != 0:
            raise CacheError(self._lib.xi_cm_last_error(self._h).decode())

    def decode_step(self, rids: np.ndarray, tokens: np.ndarray, reserve: bool, vocab: int, max_positions: int,
                    max_pages: int, rows: np.ndarray, out32: np.ndarray, out64: np.ndarray):
        """A step of one token per request prepared in one call (see xi_cm_decode_step): fills the
        two upload buffers and returns (longest cached length, lengths are similar).  Raises
        CacheError(kind, entry) for a request that cannot take part, OutOfPages if pages run out."""
        stats = np.zeros(2, np.int32)
        bad = np.zeros(1, np.int32)
        rc = self._lib.xi_cm_decode_step(
            self._h, int(rids.size), rids.ctypes.data_as(_I64P), tokens.ctypes.data_as(_I32P), int(bool(reserve)),
            int(vocab), int(max_positions), int(max_pages), rows.ctypes.data_as(_I32P), int(rows.size),
            out32.ctypes.data_as(_I32P), out64.ctypes.data_as(_I64P), stats.ctypes.data_as(_I32P),
            bad.ctypes.data_as(_I32P))
        if rc == 0:
            return int(stats[0]), bool(stats[1])
        b = int(bad[0])
        if rc == -5:
            msg = self._lib.xi_cm_last_error(self._h).decode()
            raise OutOfPages(f"request {int(rids[b])} needs pages for 1 more tokens: {msg}")
        raise DecodeStepError(rc, b)

    def release(self, rid: int) -> int:
        r = self._lib.xi_cm_release(self._h, rid)
        if r < 0:
            raise CacheError(self._lib.xi_cm_last_error(self._h).decode())
        return r

    # ---- batch arrays ---------------------------------------------------------
    def build_batch(self, rids: Sequence[int], n_tokens: Sequence[int],
                    max_pages: Optional[int] = None) -> BatchArrays:
        B = len(rids)
        T = int(np.sum(n_tokens)) if isinstance(n_tokens, np.ndarray) else int(sum(n_tokens))
        G = len(self.groups)
        ids = rids if isinstance(rids, np.ndarray) and rids.dtype == np.int64 else np.asarray(rids, dtype=np.int64)
        if max_pages is None:
            max_pages = self._lib.xi_cm_max_table_len(self._h, B, ids.ctypes.data_as(_I64P))
            if max_pages < 0:
                raise CacheError("cannot build the batch: a request is not live")
        nt = n_tokens if isinstance(n_tokens, np.ndarray) and n_tokens.dtype == np.int32 else np.asarray(n_tokens, dtype=np.int32)
        out = BatchArrays(
            num_tokens=T, num_seqs=B, max_pages=int(max_pages),
            positions=np.empty(T, np.int32), tok_seq=np.empty(T, np.int32),
            cu_q=np.empty(B + 1, np.int32), ctx_lens=np.empty(B, np.int32),
            state_slots=np.empty(B, np.int32), slots=np.empty((G, T), np.int64),
            block_tables=np.empty((G, B, int(max_pages)), np.int32))
        p32 = lambda a: a.ctypes.data_as(_I32P)
        rc = self._lib.xi_cm_build_batch(
            self._h, B, ids.ctypes.data_as(_I64P), p32(nt), p32(out.positions), p32(out.tok_seq),
            p32(out.cu_q), p32(out.ctx_lens), p32(out.state_slots),
            out.slots.ctypes.data_as(_I64P), p32(out.block_tables), int(max_pages), T)
        if rc != 0:
            why = {-1: "a request is not live", -2: "an entry has no tokens",
                   -3: "pages were not reserved for an entry", -4: "max_pages is too small",
                   -5: "a new token has no page", -6: "token count mismatch"}.get(rc, str(rc))
            raise CacheError(f"cannot build the batch: {why}")
        return out
