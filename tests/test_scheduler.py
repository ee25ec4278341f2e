"""The scheduler's decisions, as numbers (no device): admission, portions under the token
budget, decoding first, finishing, and what happens when pages run out."""
import random

import pytest

from axon_amd.engine.scheduler import Scheduler, SchedulerError


def sched(n_pages=16, page=4, window=0, budget=16, max_seqs=4, max_len=256):
    return Scheduler([n_pages], [page], [window], budget, max_seqs, max_len)


class Pool:
    """Mirrors the pages a real cache would hold, from the plans alone."""

    def __init__(self, n_pages, page):
        self.n, self.page, self.held = n_pages, page, {}

    def free(self):
        return [self.n - sum(self.held.values())]

    def grow(self, rid, n_tokens):
        self.held[rid] = max(self.held.get(rid, 0), -(-n_tokens // self.page))
        assert sum(self.held.values()) <= self.n, "the plan needs more pages than the pool has"

    def drop(self, rid):
        self.held.pop(rid, None)


def test_portions_under_the_budget_then_decode_first():
    s, pool = sched(budget=16), Pool(16, 4)
    s.add(1, 30, 4)
    plan, pre = s.plan(pool.free())
    assert [(p.id, p.start, p.count, p.wants_logits) for p in plan] == [(1, 0, 16, False)] and pre == []
    s.commit(1, 16, False, False)
    pool.grow(1, 16)
    s.add(2, 5, 4)
    plan, _ = s.plan(pool.free())                           # the older prompt first, the rest to the newcomer
    assert [(p.id, p.start, p.count, p.wants_logits) for p in plan] == [(1, 16, 14, True), (2, 0, 2, False)]
    s.commit(1, 14, True, False)
    s.commit(2, 2, False, False)
    pool.grow(1, 30), pool.grow(2, 2)
    plan, _ = s.plan(pool.free())                           # request 1 decodes now: it is served first
    assert [(p.id, p.start, p.count, p.wants_logits) for p in plan] == [(1, 30, 1, True), (2, 2, 3, True)]
    assert s.counts() == (0, 2, 0)


def test_first_come_first_served_and_slots():
    s, pool = sched(budget=64, max_seqs=2, n_pages=64), Pool(64, 4)
    for rid in (1, 2, 3):
        s.add(rid, 6, 2)
    plan, _ = s.plan(pool.free())
    assert [p.id for p in plan] == [1, 2] and s.counts()[0] == 1          # two slots: the third waits
    for p in plan:
        s.commit(p.id, p.count, True, p.id == 1)                           # 1 finishes at once
    plan, _ = s.plan(pool.free())
    assert sorted(p.id for p in plan) == [2, 3]


def test_refusals_when_added():
    s = sched(n_pages=4, page=4, max_len=40)
    with pytest.raises(SchedulerError) as e:
        s.add(1, 10, 7)                                                    # 17 tokens need 5 pages
    assert "pages" in str(e.value)
    with pytest.raises(SchedulerError):
        s.add(2, 39, 2)                                                    # beyond the positions allowed
    with pytest.raises(SchedulerError):
        s.add(3, 0, 2)
    s.add(4, 8, 8)
    with pytest.raises(SchedulerError):
        s.add(4, 8, 8)                                                     # the id is in use


def test_when_pages_run_out_the_youngest_gives_way_and_comes_back():
    s2, pool2 = sched(n_pages=5, page=4, budget=32), Pool(5, 4)
    s2.add(1, 8, 8)
    s2.add(2, 8, 8)                                                        # each fits alone (4 pages) and both start
    plan, _ = s2.plan(pool2.free())
    assert [p.id for p in plan] == [1, 2]
    for p in plan:
        s2.commit(p.id, p.count, True, False)
        pool2.grow(p.id, 8)
    steps, preempted_seen = 0, []
    out = {1: 1, 2: 1}
    while s2.counts()[0] + s2.counts()[1] > 0 and steps < 100:
        plan, pre = s2.plan(pool2.free())
        for rid in pre:
            pool2.drop(rid)
            preempted_seen.append(rid)
        assert plan, "the oldest request must always make progress"
        for p in plan:
            pool2.grow(p.id, p.start + p.count)
            done = False
            if p.wants_logits:
                out[p.id] += 1
                done = out[p.id] >= 8
            s2.commit(p.id, p.count, p.wants_logits and not done or (p.wants_logits and done), done)
            if done:
                pool2.drop(p.id)
        steps += 1
    assert out == {1: 8, 2: 8}
    assert preempted_seen and set(preempted_seen) == {2}                   # the younger one yielded, never the older
    assert s2.counts() == (0, 0, len(preempted_seen))


def test_preempted_request_is_fed_again_from_zero_with_what_it_generated():
    s, pool = sched(n_pages=5, page=4, budget=32), Pool(5, 4)
    s.add(1, 8, 8)
    s.add(2, 8, 8)
    made = {1: 0, 2: 0}
    total_when_preempted = None
    refed = None
    for _ in range(60):
        plan, pre = s.plan(pool.free())
        for rid in pre:
            pool.drop(rid)
            total_when_preempted = s.progress(rid)[1]
            assert s.progress(rid) == (0, total_when_preempted, False)      # nothing cached, back to waiting
        for p in plan:
            if total_when_preempted is not None and refed is None and p.id == 2:
                refed = (p.start, p.count, p.wants_logits)
            pool.grow(p.id, p.start + p.count)
            done = False
            if p.wants_logits:
                made[p.id] += 1
                done = made[p.id] >= 8
            s.commit(p.id, p.count, p.wants_logits, done)
            if done:
                pool.drop(p.id)
        if s.counts()[:2] == (0, 0):
            break
    assert made == {1: 8, 2: 8}
    assert total_when_preempted is not None and total_when_preempted > 8    # it had generated tokens already
    assert refed == (0, total_when_preempted, True)                         # prompt and generated tokens, in one portion


@pytest.mark.parametrize("seed", range(5))
def test_random_workloads_finish_within_the_pool(seed):
    rng = random.Random(seed)
    page = rng.choice([2, 4, 8])
    n_pages = rng.randint(12, 30)
    budget = rng.choice([8, 16, 40])
    s, pool = sched(n_pages=n_pages, page=page, budget=budget, max_seqs=4, max_len=n_pages * page), Pool(n_pages, page)
    want = {}
    rid = 0
    made = {}
    for step in range(3000):
        if rid < 25 and rng.random() < 0.3:
            prompt, new = rng.randint(1, 40), rng.randint(1, 12)
            try:
                s.add(rid, prompt, new)
                want[rid], made[rid] = new, 0
            except SchedulerError:
                assert -(-(prompt + new) // page) > n_pages
            rid += 1
        plan, pre = s.plan(pool.free())
        for r in pre:
            pool.drop(r)
        assert sum(p.count for p in plan) <= budget
        assert len({p.id for p in plan}) == len(plan)
        for p in plan:
            pool.grow(p.id, p.start + p.count)
            done = False
            if p.wants_logits:
                made[p.id] += 1
                done = made[p.id] >= want[p.id]
            s.commit(p.id, p.count, p.wants_logits, done)
            if done:
                pool.drop(p.id)
        if rid >= 25 and s.counts()[:2] == (0, 0):
            break
    assert s.counts()[:2] == (0, 0) and all(made[r] == want[r] for r in want)
