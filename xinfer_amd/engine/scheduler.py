"""Python face of the native scheduler (csrc/host/scheduler.{h,cpp})."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Tuple

from ..cache.manager import PagedCacheManager, _I32P, _I64P
from ..csrc.build import load_host


class SchedulerError(RuntimeError):
    pass


class RequestTooLarge(SchedulerError):
    """The request could not fit in the cache even alone; it was not admitted."""


@dataclass(frozen=True)
class PlannedEntry:
    request: int
    start: int        # position of the entry's first token
    count: int        # number of tokens
    sample: bool      # the entry ends at the request's last known token: sample after it


def _bind(lib):
    if getattr(lib, "_xi_sched_bound", False):
        return lib
    vp, i, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    sig = {
        "xi_sched_create": (vp, [vp, i, i, i]),
        "xi_sched_destroy": (None, [vp]),
        "xi_sched_add": (i, [vp, i64, i64, i64]),
        "xi_sched_schedule": (i, [vp, _I64P, _I64P, _I32P, _I32P, i, _I64P, i, _I32P]),
        "xi_sched_commit": (None, [vp]),
        "xi_sched_append_token": (i, [vp, i64]),
        "xi_sched_finish": (i, [vp, i64]),
        "xi_sched_num_waiting": (i, [vp]),
        "xi_sched_num_running": (i, [vp]),
        "xi_sched_computed": (i64, [vp, i64]),
        "xi_sched_last_error": (ctypes.c_char_p, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._xi_sched_bound = True
    return lib


class Scheduler:
    def __init__(self, cache: PagedCacheManager, max_num_seqs: int, max_batched_tokens: int,
                 chunk_size: int):
        self._lib = _bind(load_host())
        self.cache = cache                       # kept alive: the native scheduler points into it
        self.max_num_seqs = min(int(max_num_seqs), cache.max_requests)
        self.max_batched_tokens = int(max_batched_tokens)
        self.chunk_size = int(chunk_size)
        self._h = self._lib.xi_sched_create(cache._h, self.max_num_seqs, self.max_batched_tokens,
                                            self.chunk_size)
        if not self._h:
            raise SchedulerError("cannot create the scheduler")
        cap = self.max_num_seqs + 1
        self._ids = (ctypes.c_int64 * cap)()
        self._starts = (ctypes.c_int64 * cap)()
        self._counts = (ctypes.c_int32 * cap)()
        self._sample = (ctypes.c_int32 * cap)()
        self._pre = (ctypes.c_int64 * (4 * cap))()
        self._cap = cap

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.xi_sched_destroy(h)

    def add(self, rid: int, prompt_len: int, max_new_tokens: int) -> None:
        rc = self._lib.xi_sched_add(self._h, rid, prompt_len, max_new_tokens)
        if rc == -1:
            raise RequestTooLarge(self._lib.xi_sched_last_error(self._h).decode())
        if rc != 0:
            raise SchedulerError(self._lib.xi_sched_last_error(self._h).decode())

    def schedule(self) -> Tuple[List[PlannedEntry], List[int]]:
        """Plans one step (pages reserved).  Returns (entries, ids preempted while planning)."""
        n_pre = ctypes.c_int32(0)
        n = self._lib.xi_sched_schedule(self._h, self._ids, self._starts, self._counts, self._sample,
                                        self._cap, self._pre, 4 * self._cap, ctypes.byref(n_pre))
        if n < 0:
            raise SchedulerError("the planned step has more entries than the scheduler allows")
        entries = [PlannedEntry(self._ids[i], self._starts[i], self._counts[i], bool(self._sample[i]))
                   for i in range(n)]
        return entries, [self._pre[i] for i in range(min(n_pre.value, 4 * self._cap))]

    def commit(self) -> None:
        self._lib.xi_sched_commit(self._h)

    def append_token(self, rid: int) -> None:
        if self._lib.xi_sched_append_token(self._h, rid) != 0:
            raise SchedulerError(f"request {rid} is unknown or already at its length limit")

    def finish(self, rid: int) -> None:
        if self._lib.xi_sched_finish(self._h, rid) != 0:
            raise SchedulerError(f"request {rid} is unknown")

    def num_waiting(self) -> int:
        return self._lib.xi_sched_num_waiting(self._h)

    def num_running(self) -> int:
        return self._lib.xi_sched_num_running(self._h)

    def computed(self, rid: int) -> int:
        return self._lib.xi_sched_computed(self._h, rid)

    def idle(self) -> bool:
        return self.num_waiting() == 0 and self.num_running() == 0
