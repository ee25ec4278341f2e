"""The cache manager's bookkeeping (no device): no page lost, held twice or freed twice, under
random orders of requests; a failed reservation takes nothing; windows give pages back."""
import random

import pytest

from axon_amd.cache import CacheError, CacheManager, GroupPlan, OutOfPages
from axon_amd.parts import CacheSpec


def manager(n_pages=12, page=4, window=0, max_seqs=4, max_len=64, groups=None, seed=-1):
    groups = groups or [GroupPlan(CacheSpec(2, 2, 16, window), 2, page, n_pages)]
    return CacheManager(groups, [], max_seqs, max_len, device=None, shuffle_seed=seed)


def test_pages_follow_lengths_and_come_back():
    m = manager()
    a, b = m.open(), m.open()
    assert (a, b) == (0, 1) and m.free_slots() == 2
    m.reserve(a, 5)
    assert m.pages_of(0, a) == 2 and m.free_pages() == 10 and m.row(0, a) == [0, 1]
    m.reserve(b, 9)
    assert m.row(0, b) == [2, 3, 4]
    m.reserve(a, 8)                                          # still two pages
    assert m.pages_of(0, a) == 2
    m.reserve(a, 9)
    assert m.row(0, a) == [0, 1, 5]
    m.check()
    assert m.close(b) == 3 and m.free_pages() == 9
    c = m.open()
    assert c == b                                            # the slot is used again
    m.reserve(c, 4)
    assert m.row(0, c) == [4]                                # ... and so is the page given back last
    m.close(a), m.close(c)
    assert m.free_pages() == 12 and m.free_slots() == 4
    m.check()


def test_failed_reservation_takes_nothing():
    m = manager(n_pages=4)
    a, b = m.open(), m.open()
    m.reserve(a, 9)                                          # 3 of 4 pages
    with pytest.raises(OutOfPages) as e:
        m.reserve(b, 9)
    assert e.value.short == 2 and m.free_pages() == 1 and m.pages_of(0, b) == 0
    m.reserve(b, 4)
    m.check()
    with pytest.raises(CacheError):
        m.reserve(a, 65)                                     # beyond what a request may reach


def test_double_close_and_exhausted_slots_are_errors():
    m = manager(max_seqs=2)
    a = m.open()
    m.open()
    with pytest.raises(CacheError):
        m.open()
    m.close(a)
    with pytest.raises(CacheError):
        m.close(a)
    with pytest.raises(CacheError):
        m.close(7)
    m.check()


def test_window_gives_pages_back_and_they_are_used_again():
    m = manager(n_pages=6, page=4, window=6, max_len=200)
    a = m.open()
    held = []
    for n in range(1, 60):
        m.reserve(a, n)
        m.trim(a, n)
        held.append(m.pages_of(0, a))
        m.check()
    # the next token at position n reads [n + 1 - 6, n]: never more than 3 pages of 4
    assert max(held) <= 3 and m.free_pages() >= 3
    row = m.row(0, a)
    assert len(row) == 15 and row[0] == 0                    # given-back entries read as page 0
    m.close(a)
    assert m.free_pages() == 6


def test_groups_are_reserved_together_or_not_at_all():
    groups = [GroupPlan(CacheSpec(2, 2, 16, 0), 2, 4, 8), GroupPlan(CacheSpec(2, 1, 32, 8), 1, 8, 2)]
    m = manager(groups=groups, max_len=128)
    a = m.open()
    m.reserve(a, 16)                                         # 4 pages of group 0, 2 of group 1
    assert (m.pages_of(0, a), m.pages_of(1, a)) == (4, 2)
    with pytest.raises(OutOfPages):
        m.reserve(a, 17)                                     # group 1 is full: group 0 must stay as it was
    assert (m.pages_of(0, a), m.pages_of(1, a)) == (4, 2) and m.free_pages(0) == 4
    m.trim(a, 16)                                            # window 8: position 16 reads from 9 on
    assert m.pages_of(1, a) == 1
    m.reserve(a, 17)
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    window = rng.choice([0, 0, 5, 11])
    m = manager(n_pages=rng.randint(6, 20), page=rng.choice([1, 3, 4, 8]), window=window, max_seqs=5, max_len=96,
                seed=seed if seed % 2 else -1)
    live = {}
    for _ in range(1500):
        op = rng.random()
        if op < 0.15 and len(live) < 5:
            live[m.open()] = 0
        elif op < 0.75 and live:
            s = rng.choice(list(live))
            n = min(96, live[s] + rng.randint(1, 9))
            before = (m.free_pages(), m.pages_of(0, s))
            try:
                m.reserve(s, n)
                live[s] = n
                m.trim(s, n)
            except OutOfPages:
                assert (m.free_pages(), m.pages_of(0, s)) == before
        elif live:
            s = rng.choice(list(live))
            held = m.pages_of(0, s)
            assert m.close(s) == held
            del live[s]
        m.check()
        rows = [p for s in live for p, keep in zip(m.row(0, s), range(10 ** 6))]
        assert m.free_pages() + sum(m.pages_of(0, s) for s in live) == m.plans[0].n_pages
    for s in list(live):
        m.close(s)
    assert m.free_pages() == m.plans[0].n_pages and m.free_slots() == 5
    m.check()


def test_a_steps_reservation_is_for_all_of_its_requests_or_for_none():
    """Two live requests and a new one, the pool one page short of what the three need together:
    nothing is taken (the live requests keep exactly their pages), and with one page less to
    ask for all three get theirs."""
    spec = CacheSpec(entries=2, heads=2, head_dim=16)
    cm = CacheManager([GroupPlan(spec, 2, 8, 10)], [], 4, 256)
    a, b = cm.open(), cm.open()
    cm.reserve(a, 20)      # 3 pages
    cm.reserve(b, 9)       # 2 pages
    c = cm.open()
    free = cm.free_pages(0)
    assert free == 5
    before = [(cm.pages_of(0, s), cm.row(0, s)) for s in (a, b, c)]
    with pytest.raises(OutOfPages) as info:
        cm.reserve_many([(a, 33), (b, 17), (c, 17)])          # 2 + 1 + 3 = 6 pages, 5 free
    assert info.value.short == 1
    assert cm.free_pages(0) == free and [(cm.pages_of(0, s), cm.row(0, s)) for s in (a, b, c)] == before
    cm.check()
    cm.reserve_many([(a, 33), (b, 17), (c, 16)])              # 2 + 1 + 2
    assert cm.free_pages(0) == 0 and [cm.pages_of(0, s) for s in (a, b, c)] == [5, 3, 2]
    cm.check()
    with pytest.raises(CacheError):
        cm.reserve_many([(a, 34), (a, 35)])                    # a slot twice
    for s in (a, b, c):
        cm.close(s)
    cm.check()
    assert cm.free_pages(0) == 10
