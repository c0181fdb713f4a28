"""The scheduler's decisions (no GPU): admission, token budget, portions, decode beside
prefill, finishing and freeing, and what happens when pages run out."""
import random

import pytest

from xinfer_amd.cache import CacheGroup, PagedCacheManager
from xinfer_amd.engine.scheduler import RequestTooLarge, Scheduler, SchedulerError


def make(num_pages=64, page=16, max_seqs=4, budget=64, chunk=32, window_pages=None):
    groups = [CacheGroup(page, num_pages)]
    if window_pages:
        groups.append(CacheGroup(page, window_pages, window=20))
    cm = PagedCacheManager(groups, max_requests=max_seqs)
    return cm, Scheduler(cm, max_seqs, budget, chunk)


def drive(s, cm, reqs, max_steps=10000, on_step=None):
    """Runs the schedule/commit/append loop with made-up tokens until everything finished.
    reqs: id -> (prompt_len, max_new).  Returns per request the list of (start, count)."""
    total = {rid: p for rid, (p, _) in reqs.items()}
    new = {rid: 0 for rid in reqs}
    seen = {rid: [] for rid in reqs}
    steps = 0
    while not s.idle():
        plan, pre = s.schedule()
        assert plan, "nothing planned although requests remain"
        for rid in pre:
            seen[rid].append("preempted")
        assert sum(e.count for e in plan) <= s.max_batched_tokens
        assert len({e.request for e in plan}) == len(plan) <= s.max_num_seqs
        for e in plan:
            assert 1 <= e.count <= s.chunk_size
            assert e.start == s.computed(e.request)
            assert e.sample == (e.start + e.count == total[e.request])
            seen[e.request].append((e.start, e.count))
        if on_step:
            on_step(plan)
        s.commit()
        cm.check()
        for e in plan:
            if e.sample:
                new[e.request] += 1
                if new[e.request] >= reqs[e.request][1]:
                    s.finish(e.request)
                else:
                    total[e.request] += 1
                    s.append_token(e.request)
        steps += 1
        assert steps < max_steps
    return seen, steps


def test_portions_budget_and_mixing():
    cm, s = make(budget=40, chunk=32)
    s.add(0, 70, 3)
    s.add(1, 10, 5)
    plan, _ = s.schedule()
    # request 0 gets a portion of 32; request 1's whole prompt (10) no longer fits the 8 left
    assert [(e.request, e.start, e.count, e.sample) for e in plan] == [(0, 0, 32, False), (1, 0, 8, False)]
    s.commit()
    plan, _ = s.schedule()
    assert [(e.request, e.start, e.count, e.sample) for e in plan] == [(0, 32, 32, False), (1, 8, 2, True)]
    s.commit()
    s.append_token(1)
    plan, _ = s.schedule()
    # a decode token of request 1 is planned first, beside the last portion of request 0
    assert [(e.request, e.start, e.count, e.sample) for e in plan] == [(1, 10, 1, True), (0, 64, 6, True)]


def test_decoding_requests_come_longest_first():
    """The attention kernel's workgroups start in the batch's order; the long sequences' must not be the last."""
    cm, s = make(num_pages=64, max_seqs=4, budget=64, chunk=32)
    for rid, prompt in enumerate([5, 30, 12]):
        s.add(rid, prompt, 4)
    plan, _ = s.schedule()
    assert [(e.request, e.count) for e in plan] == [(0, 5), (1, 30), (2, 12)]      # prompts: in the queue's order
    s.commit()
    for rid in range(3):
        s.append_token(rid)
    s.add(3, 20, 4)
    plan, _ = s.schedule()
    assert [(e.request, e.start, e.count) for e in plan] == [(1, 30, 1), (2, 12, 1), (0, 5, 1), (3, 0, 20)]
    s.commit()
    for rid in range(4):
        s.append_token(rid)
    plan, _ = s.schedule()
    assert [(e.request, e.start) for e in plan] == [(1, 31), (3, 20), (2, 13), (0, 6)]


def test_every_token_is_processed_exactly_once():
    cm, s = make(num_pages=64, budget=48, chunk=20)
    reqs = {0: (70, 4), 1: (1, 9), 2: (33, 1), 3: (20, 6), 4: (47, 3), 5: (5, 5)}
    for rid, (p, n) in reqs.items():
        s.add(rid, p, n)
    seen, _ = drive(s, cm, reqs)
    for rid, (p, n) in reqs.items():
        spans = [x for x in seen[rid] if x != "preempted"]
        pos = 0
        for start, count in spans:
            assert start == pos
            pos += count
        assert pos == p + n - 1            # the last sampled token is never fed
    assert cm.free_pages(0) == 64 and cm.live_requests() == 0


def test_max_num_seqs_limits_admission():
    cm, s = make(max_seqs=2, budget=1000, chunk=1000)
    for rid in range(5):
        s.add(rid, 8, 2)
    plan, _ = s.schedule()
    assert [e.request for e in plan] == [0, 1] and s.num_waiting() == 3


def test_request_that_can_never_fit_is_refused():
    cm, s = make(num_pages=4, page=16)
    with pytest.raises(RequestTooLarge, match="cache pages"):
        s.add(0, 60, 8)                    # 68 tokens need 5 pages
    s.add(1, 60, 4)                        # 64 tokens fit exactly
    with pytest.raises(SchedulerError, match="exists"):
        s.add(1, 3, 3)
    with pytest.raises(SchedulerError):
        s.add(2, 0, 3)


def test_admission_waits_for_pages():
    cm, s = make(num_pages=6, page=16, budget=1000, chunk=1000)
    s.add(0, 64, 16)                       # 4 pages now, a fifth later
    s.add(1, 48, 4)                        # needs 3 pages: only 2 are left
    plan, _ = s.schedule()
    assert [e.request for e in plan] == [0] and s.num_waiting() == 1
    s.commit()
    s.finish(0)
    plan, _ = s.schedule()
    assert [e.request for e in plan] == [1] and cm.free_pages(0) == 3


def test_out_of_pages_preempts_the_youngest_and_recomputes():
    """Two requests fill the pool; when the older one needs another page the younger one is
    preempted, waits at the head of the queue, and is later recomputed from its first token
    (prompt and generated tokens alike)."""
    cm, s = make(num_pages=4, page=16, budget=1000, chunk=1000)
    reqs = {0: (30, 10), 1: (31, 20)}
    for rid, (p, n) in reqs.items():
        s.add(rid, p, n)
    seen, _ = drive(s, cm, reqs)
    assert "preempted" in seen[1] and "preempted" not in seen[0]
    i = seen[1].index("preempted")
    before, after = seen[1][:i], seen[1][i + 1:]
    assert before[0] == (0, 31) and all(c == 1 for _, c in before[1:])
    assert after[0][0] == 0 and after[0][1] == 31 + len(before) - 1 + 1   # all known tokens again
    assert cm.free_pages(0) == 4


@pytest.mark.parametrize("seed", range(5))
def test_random_workloads_finish_and_free_everything(seed):
    rng = random.Random(seed)
    cm, s = make(num_pages=rng.choice([12, 20, 40]), page=rng.choice([4, 8, 16]), max_seqs=rng.choice([2, 4]),
                 budget=rng.choice([16, 33, 64]), chunk=rng.choice([5, 16, 48]), window_pages=rng.choice([None, 40]))
    cap = cm.groups[0].num_pages * cm.groups[0].page_size
    reqs = {}
    for rid in range(12):
        p = rng.randrange(1, cap // 2)
        n = rng.randrange(1, max(2, min(30, cap - p)))
        reqs[rid] = (p, n)
        s.add(rid, p, n)
    seen, steps = drive(s, cm, reqs)
    assert cm.live_requests() == 0
    for g, grp in enumerate(cm.groups):
        assert cm.free_pages(g) == grp.num_pages


def test_a_window_group_holds_the_window_and_a_portion_not_the_whole_request():
    """A prompt of 400 tokens on a model with a group that keeps the last 20 keys: that group's pool
    of 5 pages of 16 tokens (window - 1 + a portion of 32 = 51 tokens, 4 pages, and one more for a start
    inside a page) is enough, while the group that keeps every key needs all 26.  The request is
    admitted, runs in portions without a preemption, and the window group never holds more than
    its 5 pages; with 4 it is refused when added."""
    cm, s = make(num_pages=26, page=16, max_seqs=2, budget=32, chunk=32, window_pages=5)
    s.add(0, 400, 8)
    most = [0]

    def on_step(plan):
        most[0] = max(most[0], 5 - cm.free_pages(1))
    seen, steps = drive(s, cm, {0: (400, 8)}, on_step=on_step)
    assert "preempted" not in seen[0]
    assert [c for _, c in seen[0][:13]] == [32] * 12 + [16] and steps == 13 + 7
    assert 4 <= most[0] <= 5
    assert cm.free_pages(0) == 26 and cm.free_pages(1) == 5
    cm, s = make(num_pages=26, page=16, max_seqs=2, budget=32, chunk=32, window_pages=4)
    with pytest.raises(RequestTooLarge):
        s.add(0, 400, 8)
    s.add(1, 40, 8)             # 48 tokens at most: 3 pages hold them all


def test_two_long_requests_share_a_small_window_pool():
    """Two requests whose window pages would not fit if each held its whole length: both run to the
    end; when the window pool is short the younger gives way and is recomputed."""
    cm, s = make(num_pages=60, page=16, max_seqs=2, budget=48, chunk=24, window_pages=7)
    reqs = {0: (300, 20), 1: (250, 30)}
    for rid, (p, n) in reqs.items():
        s.add(rid, p, n)
    seen, _ = drive(s, cm, reqs)
    for rid, (p, n) in reqs.items():
        spans = [x for x in seen[rid] if x != "preempted"]
        assert spans[-1][0] + spans[-1][1] == p + n - 1
    assert cm.free_pages(0) == 60 and cm.free_pages(1) == 7


@pytest.mark.parametrize("seed", range(6))
def test_running_one_step_ahead_keeps_the_books(seed):
    """The engine's way of running ahead, with made-up tokens: after a step is committed every
    sampled request is told to grow by one (or, if that token is the last its length allows, let go
    of at once), the next step is planned and committed, and only then does the loop learn which
    requests of the step before ended on their token's value; those are finished late, after one more
    token of theirs has run for nothing.  Under random sizes, few pages (requests are preempted with
    a token still on its way) and a window group: plans stay consistent, every request runs all its
    tokens, and every page and slot comes back."""
    rng = random.Random(100 + seed)
    cm, s = make(num_pages=rng.choice([10, 16, 40]), page=rng.choice([4, 8, 16]), max_seqs=rng.choice([2, 3, 4]),
                 budget=rng.choice([16, 33, 64]), chunk=rng.choice([5, 16, 48]), window_pages=rng.choice([None, 40]))
    cap = cm.groups[0].num_pages * cm.groups[0].page_size
    reqs, ends_at = {}, {}
    for rid in range(14):
        p = rng.randrange(1, cap // 2)
        n = rng.randrange(1, max(2, min(30, cap - p)))
        reqs[rid] = (p, n)
        ends_at[rid] = rng.randrange(1, n + 1) if rng.random() < 0.6 else None     # its k-th token is an end-of-sequence
        s.add(rid, p, n)
    total = {rid: p for rid, (p, _) in reqs.items()}        # tokens the scheduler knows of
    sampled_n = {rid: 0 for rid in reqs}                     # tokens sampled for it (launched)
    live, closed, preempted_n, wasted = set(reqs), set(), 0, 0
    launched = None                                          # requests sampled by the step that is "on the GPU"
    steps = 0
    while not s.idle() or launched:
        plan, pre = s.schedule()
        preempted_n += len(pre)
        if launched and not plan:
            pass                                             # nothing to launch: only the earlier step is read
        else:
            assert plan, "nothing planned although requests remain"
            assert sum(e.count for e in plan) <= s.max_batched_tokens
            assert len({e.request for e in plan}) == len(plan) <= s.max_num_seqs
            for e in plan:
                assert e.request in live and e.request not in closed
                assert e.start == s.computed(e.request) and e.sample == (e.start + e.count == total[e.request])
            s.commit()
            cm.check()
        now = []
        for e in plan:
            if e.sample:
                rid = e.request
                sampled_n[rid] += 1
                now.append((rid, sampled_n[rid]))
                if sampled_n[rid] >= reqs[rid][1]:           # its last token by length: the scheduler lets go now
                    s.finish(rid)
                    closed.add(rid)
                else:
                    total[rid] += 1
                    s.append_token(rid)
        for rid, k in launched or []:                        # the step before is read now
            if rid not in live:
                wasted += 1                                  # it ended a step ago: this token ran for nothing
                continue
            if ends_at[rid] == k or k >= reqs[rid][1]:
                if rid not in closed:
                    s.finish(rid)
                live.discard(rid)
        launched = now
        steps += 1
        assert steps < 20000
    assert not live and cm.live_requests() == 0
    for g, grp in enumerate(cm.groups):
        assert cm.free_pages(g) == grp.num_pages
    assert wasted <= sum(1 for rid in reqs if ends_at[rid] is not None)


def test_pages_are_planned_group_by_group():
    """A group with a window gets pages for a window and a portion a request (what the scheduler
    admits it with), not for the model's whole length; if memory is short every group keeps the
    same share of what it could use; and the scheduler admits a full house on what was planned."""
    from xinfer_amd.engine.llm_engine import plan_pages
    page, seqs, length, portion = 16, 4, 4096, 64
    full, windowed = (0, 1000), (24, 500)
    got = plan_pages([full, windowed], page, seqs, length, portion, budget_bytes=1 << 40)
    assert got == [seqs * (length // page), seqs * (-(-(24 - 1 + portion) // page) + 1)] == [1024, 28]
    # a window longer than the model's length changes nothing
    assert plan_pages([(10 ** 6, 500)], page, seqs, length, portion, 1 << 40) == [1024]
    # short of memory: the same share of both, within a page
    need = 1024 * 1000 * page + 28 * 500 * page
    half = plan_pages([full, windowed], page, seqs, length, portion, need // 2)
    assert half == [512, 14]
    assert plan_pages([full, windowed], page, seqs, length, portion, 1) == [1, 1]
    assert plan_pages([], page, seqs, length, portion, 1 << 40) == [1]
    # what was planned is what the scheduler needs for max_num_seqs requests of the full length:
    # all are admitted together and nothing is ever preempted
    cm = PagedCacheManager([CacheGroup(page, got[0]), CacheGroup(page, got[1], window=24)], max_requests=seqs)
    s = Scheduler(cm, seqs, seqs * portion, portion)       # a step's budget takes a portion of every request
    for rid in range(seqs):
        s.add(rid, length - 8, 8)
    most = [0]

    def on_step(plan):
        most[0] = max(most[0], cm.live_requests())

    seen, _ = drive(s, cm, {rid: (length - 8, 8) for rid in range(seqs)}, on_step=on_step)
    assert most[0] == seqs and not any("preempted" in v for v in seen.values())
    assert cm.free_pages(0) == got[0] and cm.free_pages(1) == got[1]
