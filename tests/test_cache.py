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
    # a pool made for windows: what the requests hold at once when a step brings at most 8 tokens; without that bound,
    # or without a window, or when the whole context is shorter than that, a page for every token
    assert g.pool_pages(1000, 3, 8) == 3 * (g.pages_for(14) + 1) and g.pool_pages(1000, 3, None) == 250
    assert GroupSpec("all", 4, 64).pool_pages(1000, 3, 8) == 250 and g.pool_pages(12, 3, 8) == 3


def test_a_pool_made_for_windows_is_enough_for_steps_within_the_bound():
    """Three requests decode and take portions of at most 8 tokens through a windowed pool of pool_pages(...) pages:
    no step runs out of pages, in any interleaving tried."""
    g = GroupSpec("win", 4, 0, window=6)
    pages = g.pool_pages(10_000, 3, 8)
    rng = random.Random(5)
    m = CacheManager([GroupSpec("win", 4, pages, window=6)], max_requests=3)
    for r in "abc":
        m.open(r)
    for _ in range(600):
        r = rng.choice("abc")
        m.prepare(r, rng.choice([1, 1, 2, 5, 8]))
        m.commit(r)
        assert m.pages_in_use(0) <= pages


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    groups = [GroupSpec("kv", 4, 40), GroupSpec("win", 8, 12, window=20)]
    shadows = seed % 2 == 1
    m = CacheManager(groups, max_requests=5, shadow_slots=shadows)
    live, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            m.open(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.35 and live:
            r = rng.choice(list(live))
            to = rng.randint(0, live[r])
            try:
                m.truncate(r, to)
            except CacheLogicError as e:
                assert "keeps the last 20 keys only" in str(e) and m.length(r) == live[r]
            else:
                live[r] = to
                assert m.length(r) == to and m.pages_held(r, 0) == -(-to // 4)
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
        assert all(m.step_slot(r) == m.slot(r) for r in live)      # no step is in progress: nobody holds a second slot
    for r in list(live):
        m.close(r)
    assert all(m.pages_in_use(g) == 0 for g in range(2)) and m.slots.in_use == 0
    m.open("after")
    m.prepare("after", 40 * 4 if False else 12 * 8)        # a request as long as the smaller pool: every page came back
    m.commit("after")


def test_truncate_returns_the_pages_beyond_the_new_length():
    """/root/reference/src/model/kv_cache.hpp:126-134: the history is rolled back to `length` and the blocks beyond it
    go back; reset is truncate(0)."""
    m = CacheManager([GroupSpec("kv", 4, 10)], max_requests=2)
    m.open("a")
    m.prepare("a", 18)
    m.commit("a")
    held = list(m.table("a", 0))
    assert m.pages_in_use() == 5
    m.truncate("a", 18)                                   # to its own length: nothing changes
    assert m.table("a", 0) == held
    m.truncate("a", 9)                                    # position 8 lies in the third page: it stays, two go back
    assert m.length("a") == 9 and m.table("a", 0) == held[:3] and m.pages_in_use() == 3
    m.prepare("a", 4)                                     # the request goes on from there, first with the freed pages
    m.commit("a")
    assert m.length("a") == 13 and m.table("a", 0)[:3] == held[:3] and set(m.table("a", 0)) <= set(held)
    with pytest.raises(CacheLogicError, match="holds 13 tokens and cannot be taken back to 14"):
        m.truncate("a", 14)
    with pytest.raises(CacheLogicError, match="cannot be taken back to -1"):
        m.truncate("a", -1)
    m.prepare("a", 1)
    with pytest.raises(CacheLogicError, match="step in progress"):
        m.truncate("a", 2)
    m.abort("a")
    m.truncate("a", 0)
    assert m.length("a") == 0 and m.table("a", 0) == [] and m.pages_in_use() == 0
    with pytest.raises(CacheLogicError, match="not open"):
        m.truncate("b", 0)


def test_truncate_inside_a_window_that_gave_pages_back_is_refused():
    m = CacheManager([GroupSpec("all", 4, 64), GroupSpec("win", 4, 64, window=6)], max_requests=1)
    m.open("r")
    m.prepare("r", 30)
    m.commit("r")                       # the window group holds the pages of positions 24.. only
    before = (m.length("r"), list(m.table("r", 0)), list(m.table("r", 1)))
    assert m.table("r", 1)[:6] == [-1] * 6
    with pytest.raises(CacheLogicError, match="win keeps the last 6 keys only and has given back the page of position 16"):
        m.truncate("r", 22)             # a row at 22 reads keys 17..21
    assert (m.length("r"), m.table("r", 0), m.table("r", 1)) == before       # the refusal changed nothing, in either group
    m.truncate("r", 29)                 # a row at 29 reads 24..28: still held
    assert m.length("r") == 29 and m.pages_held("r", 0) == 8
    m.truncate("r", 0)                  # to nothing is always possible
    assert m.pages_in_use(0) == 0 and m.pages_in_use(1) == 0


def test_shadow_slots_keep_the_committed_state_apart_from_a_running_step():
    """With shadow slots a step writes a second slot; commit makes it the request's, abort drops it (the reference keeps
    the live slot as a mark while a pass writes another: /root/reference/src/model/kv_cache.hpp:216-266)."""
    m = CacheManager([GroupSpec("kv", 4, 8)], max_requests=2, shadow_slots=True)
    assert m.slots.capacity == 4
    a = m.open("a")
    m.open("b")
    with pytest.raises(OutOfPages, match="every request slot is taken"):
        m.open("c")                                       # two requests at most, however many slots there are
    assert m.step_slot("a") == a
    m.prepare("a", 3)
    shadow = m.step_slot("a")
    assert shadow != a and m.slot("a") == a and m.slots.in_use == 3
    m.abort("a")
    assert m.slot("a") == a and m.step_slot("a") == a and m.slots.in_use == 2
    m.prepare("a", 3)
    shadow = m.step_slot("a")
    m.commit("a")
    assert m.slot("a") == shadow and m.slots.in_use == 2  # the old slot went back
    m.prepare("a", 1)
    m.prepare("b", 1)
    assert len({m.step_slot("a"), m.step_slot("b"), m.slot("a"), m.slot("b")}) == 4
    m.close("a")                                          # ending a request during its step gives both slots back
    m.abort("b")
    m.close("b")
    assert m.slots.in_use == 0 and m.pages_in_use() == 0
    with pytest.raises(OutOfPages):
        full = CacheManager([GroupSpec("kv", 4, 1)], max_requests=1, shadow_slots=True)
        full.open("x")
        full.prepare("x", 9)
    assert full.slots.in_use == 1 and full.step_slot("x") == full.slot("x")   # the failed prepare took no second slot
