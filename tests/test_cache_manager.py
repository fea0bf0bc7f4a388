"""The cache manager: no page lost, held twice or freed twice, under random orders of requests; windows give pages
back early; state slots.  CPU only.  The first four tests hold the vectors of the reference's tests/test_allocator.py."""

import random

import pytest

from nanospec_amd.cache import RELEASED, CacheManager, GroupSpec, PagePool, PoolExhausted, SlotPool


def one_group(pages, page, slots=8):
    return CacheManager([GroupSpec("all")], pages, page, slots)


def test_reserve_commit_release_roundtrip():
    """reference tests/test_allocator.py:8-18: 5 tokens on pages of 4 -> 2 pages; 3 more fill them; 1 more crosses."""
    m = one_group(8, 4)
    rc = m.admit(0)
    m.reserve(0, 5), m.commit(0, 5)
    assert len(rc.tables[0]) == 2
    m.reserve(0, 3), m.commit(0, 3)
    assert len(rc.tables[0]) == 2
    m.reserve(0, 1), m.commit(0, 1)
    assert len(rc.tables[0]) == 3 and rc.length == 9
    m.release(0)
    assert m.num_free() == 8
    m.check()


def test_pages_are_handed_out_from_zero_and_reused_last_in_first_out():
    """reference kv/allocator.py:27,46,72."""
    m = one_group(8, 4)
    m.admit("a"), m.reserve("a", 12)
    assert m.get("a").tables[0] == [0, 1, 2]
    m.admit("b"), m.reserve("b", 4)
    m.release("a")
    m.admit("c"), m.reserve("c", 8)
    assert m.get("c").tables[0] == [2, 1]  # the pages the finished request gave back last come first


def test_exhaustion_raises_and_leaves_state_intact():
    """reference tests/test_allocator.py:36-44."""
    m = one_group(4, 2)
    m.admit(0), m.reserve(0, 6)
    m.admit(1)
    with pytest.raises(PoolExhausted):
        m.reserve(1, 3)
    m.check()
    assert m.num_free() == 1 and m.get(1).tables[0] == [] and m.get(1).reserved == 0
    m.reserve(1, 2)
    m.check()


def test_reserve_twice_takes_nothing_more():
    m = one_group(8, 4)
    m.admit(0)
    m.reserve(0, 6), m.reserve(0, 6)
    assert m.num_free() == 6
    m.commit(0, 6)
    with pytest.raises(ValueError):
        m.commit(0, 3)  # more written than reserved


def test_double_free_and_foreign_pages_are_refused():
    pool = PagePool(4, 2)
    got = pool.take(2)
    pool.give(got)
    with pytest.raises(ValueError):
        pool.give(got[:1])
    with pytest.raises(ValueError):
        pool.give([9])
    with pytest.raises(ValueError):
        pool.give([*pool.take(1)] * 2)
    slots = SlotPool(1)
    s = slots.take()
    with pytest.raises(PoolExhausted):
        slots.take()
    slots.give(s)
    with pytest.raises(ValueError):
        slots.give(s)


def test_window_group_gives_pages_back_while_running():
    """Pages of 4, window 6: a query at position p sees p-5..p, so the page of positions 0..3 is let go once 10
    positions are written (the next query, at 10, sees 5..10)."""
    m = CacheManager([GroupSpec("all"), GroupSpec("win", window=6)], 16, 4, 4)
    rc = m.admit("r")
    m.reserve("r", 9), m.commit("r", 9)   # next query at 9 sees 4..9: page 0 (0..3) goes
    assert rc.tables[1][0] == RELEASED and rc.tables[1][1] != RELEASED
    assert all(p != RELEASED for p in rc.tables[0])
    assert m.num_free(1) == 16 - 2 and m.num_free(0) == 16 - 3
    m.reserve("r", 8), m.commit("r", 8)   # 17 written: next query at 17 sees 12..17 -> pages 0..2 gone
    assert rc.tables[1][:3] == [RELEASED] * 3 and rc.held[1] == 2
    m.check()
    m.release("r")
    assert m.num_free(0) == m.num_free(1) == 16
    m.check()
    assert m.worst_case_pages(100) == [25, 4]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_in_one_place(seed):
    """reference tests/test_allocator.py:47-75, with two groups, state slots and window releases."""
    rng = random.Random(seed)
    m = CacheManager([GroupSpec("all"), GroupSpec("win", window=rng.choice([5, 16, 33]))], [64, 24], rng.choice([4, 8, 16]), 6)
    live, next_id = [], 0
    for _ in range(500):
        op = rng.random()
        try:
            if live and op < 0.25:
                m.release(live.pop(rng.randrange(len(live))))
            elif live and op < 0.75:
                r = rng.choice(live)
                n = rng.randint(1, 40)
                m.reserve(r, n)
                m.commit(r, rng.randint(0, n))
            else:
                m.admit(next_id)
                live.append(next_id)
                next_id += 1
        except PoolExhausted:
            pass
        m.check()
    for r in live:
        m.release(r)
    m.check()
    assert m.num_free(0) == 64 and m.num_free(1) == 24 and m.slots.num_free == 6


def test_freed_pages_land_scattered():
    """After churn a new request's pages are not one contiguous run (reference tests/test_allocator.py:70-75)."""
    rng = random.Random(0)
    m = one_group(256, 16, slots=64)
    live = []
    for i in range(300):
        try:
            if live and rng.random() < 0.45:
                m.release(live.pop(rng.randrange(len(live))))
            else:
                m.admit(i), m.reserve(i, rng.randint(1, 100))
                live.append(i)
        except PoolExhausted:
            m.release(i) if i in m else None
    for r in live[: len(live) // 2]:
        m.release(r)
    m.admit("probe"), m.reserve("probe", 16 * 8)
    t = m.get("probe").tables[0]
    assert any(b != a + 1 for a, b in zip(t, t[1:])), t
    m.check()
