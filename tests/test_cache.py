"""The cache manager: no page lost, held twice or freed twice, under random orders of requests; windows; slots.
Rules of the pool follow /root/reference/tests/kv_cache.cpp:42-120 (ids dense from zero, the freed id reused first,
double release / retain of a free page / exhaustion refused, a failed prepare leaves the request unchanged)."""

import random

import pytest

from llmx_amd.cache import CacheLogicError, CacheManager, GroupSpec, OutOfPages, PagePool, StateSlots


def test_pool_rules():
    pool = PagePool(3)
    assert [pool.alloc(), pool.alloc()] == [0, 1]          # dense from zero
    pool.release(0)
    assert pool.alloc() == 0                               # the freed id first
    assert pool.alloc() == 2
    with pytest.raises(OutOfPages, match="budget exhausted"):
        pool.alloc()
    pool.release(1)
    with pytest.raises(CacheLogicError, match="released twice"):
        pool.release(1)
    with pytest.raises(CacheLogicError, match="retain of free page"):
        pool.retain(1)
    pool.retain(2)
    pool.release(2)
    assert pool.refs(2) == 1 and pool.in_use == 2 and pool.available == 1


def test_slots():
    s = StateSlots(2)
    a, b = s.alloc(), s.alloc()
    assert {a, b} == {0, 1}
    with pytest.raises(OutOfPages):
        s.alloc()
    s.release(a)
    with pytest.raises(CacheLogicError):
        s.release(a)
    assert s.alloc() == a


def test_prepare_commit_abort():
    m = CacheManager([GroupSpec("kv", 4, 5)], max_requests=2)
    m.open("a")
    m.prepare("a", 6)                      # 2 pages
    assert m.length("a") == 0 and m.pages_in_use() == 2      # prepare does not commit
    m.commit("a")
    assert m.length("a") == 6
    m.prepare("a", 1)                      # position 6 lies in the second page: nothing new
    assert m.pages_in_use() == 2
    m.abort("a")
    assert m.length("a") == 6 and m.pages_in_use() == 2
    m.open("b")
    with pytest.raises(OutOfPages):
        m.prepare("b", 13)                 # needs 4 of the 3 pages left
    assert m.pages_in_use() == 2 and m.length("b") == 0 and m.table("b", 0) == []   # the failed prepare left nothing
    m.prepare("b", 12)
    with pytest.raises(CacheLogicError, match="already has a step"):
        m.prepare("b", 1)
    m.abort("b")
    assert m.pages_in_use() == 2
    m.close("a")
    m.close("b")
    assert m.pages_in_use() == 0 and m.slots.in_use == 0
    with pytest.raises(CacheLogicError, match="not open"):
        m.length("a")


def test_window_gives_pages_back_as_it_passes_them():
    m = CacheManager([GroupSpec("all", 4, 64), GroupSpec("win", 4, 64, window=6)], max_requests=1)
    m.open("r")
    for step in range(40):
        m.prepare("r", 1)
        m.commit("r")
        L = m.length("r")
        assert m.pages_held("r", 0) == -(-L // 4)
        table = m.table("r", 1)
        # every key a later row can read (positions >= L - 6 + 1 ... wait: the next row sits at L and reads L-5 .. L) is still held
        for pos in range(max(0, L - 5), L):
            assert table[pos // 4] >= 0
        # and nothing wholly behind the window is
        for i, page in enumerate(table):
            if (i + 1) * 4 <= L - 6 + 1:
                assert page == -1
        assert m.pages_held("r", 1) <= 3
    m.close("r")
    assert m.pages_in_use(0) == 0 and m.pages_in_use(1) == 0
    g = GroupSpec("win", 4, 64, window=6)
    assert g.peak_pages(1000, 8) == g.pages_for(14) + 1 and GroupSpec("all", 4, 64).peak_pages(1000, 8) == 250


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    groups = [GroupSpec("kv", 4, 40), GroupSpec("win", 8, 12, window=20)]
    m = CacheManager(groups, max_requests=5)
    live, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            m.open(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.85 and live:
            r = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 16])
            try:
                m.prepare(r, n)
            except OutOfPages:
                assert m.length(r) == live[r]
            else:
                if rng.random() < 0.15:
                    m.abort(r)
                else:
                    m.commit(r)
                    live[r] += n
                assert m.length(r) == live[r]
        elif live:
            r = rng.choice(list(live))
            m.close(r)
            del live[r]
        # invariants: every held page is held by exactly one request; counts agree with the pools
        for gi, g in enumerate(groups):
            held = [p for r in live for p in m.table(r, gi) if p >= 0]
            assert len(held) == len(set(held)), "a page is held twice"
            assert len(held) == m.pages_in_use(gi), "a page was lost"
            assert all(0 <= p < g.n_pages for p in held)
        assert m.slots.in_use == len(live)
        assert len({m.slot(r) for r in live}) == len(live)
    for r in list(live):
        m.close(r)
    assert all(m.pages_in_use(g) == 0 for g in range(2)) and m.slots.in_use == 0
    m.open("after")
    m.prepare("after", 40 * 4 if False else 12 * 8)        # a request as long as the smaller pool: every page came back
    m.commit("after")
