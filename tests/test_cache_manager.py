"""The cache manager under random orders of requests: no page lost, held twice or freed
twice; pages come back at the end of a request and when a window has passed them, and are
handed out again (no GPU)."""
import random

import pytest

import numpy as np

from xinfer_amd.cache import CacheError, CacheGroup, DecodeStepError, OutOfPages, PagedCacheManager


def test_pages_slots_and_tables():
    cm = PagedCacheManager([CacheGroup(16, 8)], max_requests=2)
    assert cm.add_request(5) == 0 and cm.add_request(9) == 1
    with pytest.raises(CacheError, match="live already"):
        cm.add_request(5)
    with pytest.raises(CacheError, match="state slot"):
        cm.add_request(11)
    cm.reserve(5, 17)
    assert cm.block_table(5) == [0, 1] and cm.free_pages() == 6       # FIFO from the front
    b = cm.build_batch([5], [17])
    assert b.positions.tolist() == list(range(17))
    assert b.slots[0].tolist() == list(range(17))                      # page 0 then page 1
    assert b.ctx_lens.tolist() == [17] and b.cu_q.tolist() == [0, 17]
    cm.commit(5, 17)
    cm.reserve(5, 1)                                                   # token 17 fits page 1
    assert cm.block_table(5) == [0, 1]
    assert cm.build_batch([5], [1]).slots[0].tolist() == [17]
    cm.commit(5, 1)
    cm.reserve(9, 16)
    assert cm.block_table(9) == [2]
    cm.commit(9, 16)
    cm.reserve(9, 1)                                                   # position 16 opens a page
    assert cm.block_table(9) == [2, 3]
    assert cm.release(5) == 2
    cm.check()
    # pages 0 and 1 went to the back of the list and come out again after 4..7
    cm.add_request(6)
    cm.reserve(6, 16 * 6)
    assert cm.block_table(6) == [4, 5, 6, 7, 0, 1]
    cm.check()


def test_decode_step_in_one_call_matches_the_builder():
    """The one-call preparation of a step of single tokens fills the two upload buffers with
    what reserve + build_batch give, in the runner's order, and refuses what the step function
    refuses."""
    def manager():
        cm = PagedCacheManager([CacheGroup(8, 12), CacheGroup(8, 12, window=10)], max_requests=3)
        for rid, n in ((4, 13), (7, 1), (2, 24)):
            cm.add_request(rid)
            cm.reserve(rid, n)
            cm.commit(rid, n)
        return cm
    a, b = manager(), manager()
    rids = np.array([7, 2, 4], np.int64)
    toks = np.array([3, 250, 0], np.int32)
    B, G, P = 3, 2, 5
    out32 = np.full(6 * B + 1 + G * B * P, -7, np.int32)
    out64 = np.full((2 + G) * B, -7, np.int64)
    longest, similar = a.decode_step(rids, toks, True, 256, 64, P, np.array([2, 0], np.int32), out32, out64)
    b.reserve_many(rids, np.ones(B, np.int32))
    w = b.build_batch(rids, np.ones(B, np.int32), max_pages=P)
    assert longest == 25 and not similar and [a.block_table(r, g) for r in (7, 2, 4) for g in (0, 1)] == \
        [b.block_table(r, g) for r in (7, 2, 4) for g in (0, 1)]
    want32 = np.concatenate([toks, w.positions, w.tok_seq, w.cu_q, w.ctx_lens, [2, 0, 0], w.block_tables.reshape(-1)])
    want64 = np.concatenate([w.state_slots.astype(np.int64), w.slots.reshape(-1), [-1, -1, -1]])
    assert out32.tolist() == want32.tolist() and out64.tolist() == want64.tolist()
    a.commit_many(rids, np.ones(B, np.int32))
    assert a.lengths(np.array([4, 7, 2, 99], np.int64)).tolist() == [14, 2, 25, -1]
    a.check()
    assert a.decode_step(np.array([4, 7, 2], np.int64), toks, True, 256, 64, P, np.array([], np.int32), out32, out64)[1] is False
    for bad_rids, bad_toks, max_pos, rows, kind, entry in (
            ([7, 99, 4], [1, 1, 1], 64, [0], -1, 1), ([7, 2, 7], [1, 1, 1], 64, [0], -2, 2),
            ([7, 2, 4], [1, 1, 1], 25, [0], -3, 1), ([7, 2, 4], [1, 256, 1], 64, [0], -4, 1),
            ([7, 2, 4], [1, 1, 1], 64, [3], -6, 0)):
        with pytest.raises(DecodeStepError) as e:
            a.decode_step(np.array(bad_rids, np.int64), np.array(bad_toks, np.int32), True, 256, max_pos, P,
                          np.array(rows, np.int32), out32, out64)
        assert (e.value.kind, e.value.entry) == (kind, entry)
    small = PagedCacheManager([CacheGroup(8, 1)], max_requests=2)
    for rid in (0, 1):
        small.add_request(rid)
    small.reserve(0, 8)
    small.commit(0, 8)
    with pytest.raises(OutOfPages):
        small.decode_step(np.array([0], np.int64), np.array([1], np.int32), True, 256, 64, 4, np.array([0], np.int32),
                          np.zeros(11, np.int32), np.zeros(3, np.int64))


def test_reserve_is_all_or_nothing():
    cm = PagedCacheManager([CacheGroup(8, 4), CacheGroup(8, 2, window=4)], max_requests=2)
    cm.add_request(1)
    with pytest.raises(OutOfPages, match="No free blocks"):
        cm.reserve(1, 17)                     # needs 3 pages; the second group has 2
    assert cm.free_pages(0) == 4 and cm.free_pages(1) == 2 and cm.block_table(1, 0) == []
    cm.check()
    with pytest.raises(CacheError, match="cannot hold"):
        cm.commit(1, 1)                       # nothing reserved


def test_window_pages_are_given_back_while_running():
    cm = PagedCacheManager([CacheGroup(8, 16), CacheGroup(8, 16, window=10)], max_requests=1)
    cm.add_request(0)
    cm.reserve(0, 30)
    cm.commit(0, 30)
    # the next query (position 30) sees keys 21..30: pages 0 and 1 (keys 0..15) are passed
    assert cm.block_table(0, 1)[:2] == [-1, -1] and cm.block_table(0, 1)[2] >= 0
    assert cm.free_pages(1) == 16 - 2 and cm.free_pages(0) == 16 - 4
    for _ in range(40):
        cm.reserve(0, 1)
        cm.commit(0, 1)
        cm.check()
    held = [p for p in cm.block_table(0, 1) if p >= 0]
    assert len(held) <= 3                      # a window of 10 spans at most 3 pages of 8
    full = len(cm.block_table(0, 0))
    assert full == -(-70 // 8)                 # the group that keeps every key gave nothing back
    assert cm.release(0) == len(held) + full
    cm.check()
    assert cm.free_pages(0) == 16 and cm.free_pages(1) == 16


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    groups = [CacheGroup(rng.choice([4, 8, 16]), 24), CacheGroup(8, 12, window=rng.choice([5, 16, 20]))]
    cm = PagedCacheManager(groups, max_requests=4)
    live = {}
    next_id = 0
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and len(live) < 4:
            cm.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 7, 30])
            before = [cm.free_pages(g) for g in range(2)]
            try:
                cm.reserve(rid, n)
            except OutOfPages:
                assert [cm.free_pages(g) for g in range(2)] == before      # nothing changed
            else:
                b = cm.build_batch([rid], [n])
                for g, grp in enumerate(groups):
                    table = cm.block_table(rid, g)
                    for i, s in enumerate(b.slots[g].tolist()):
                        pos = live[rid] + i
                        assert s == table[pos // grp.page_size] * grp.page_size + pos % grp.page_size
                cm.commit(rid, n)
                live[rid] += n
                assert cm.length(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            cm.release(rid)
            del live[rid]
            with pytest.raises(CacheError):
                cm.release(rid)                                              # not freed twice
        cm.check()                                                           # no page lost or held twice
        # no physical page in two live tables
        for g in range(2):
            seen = set()
            for rid in live:
                for p in cm.block_table(rid, g):
                    if p >= 0:
                        assert p not in seen
                        seen.add(p)
            assert len(seen) + cm.free_pages(g) == groups[g].num_pages
    for rid in list(live):
        cm.release(rid)
    cm.check()
    assert [cm.free_pages(g) for g in range(2)] == [24, 12] and cm.free_state_slots() == 4
