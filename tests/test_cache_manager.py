"""The cache manager under random orders of requests: no page lost, held twice or freed
twice; pages come back at the end of a request and when a window has passed them, and are
handed out again (no GPU)."""
import random

import pytest

from xinfer_amd.cache import CacheError, CacheGroup, OutOfPages, PagedCacheManager


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
