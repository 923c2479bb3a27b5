"""The cache manager on the host: no page lost, held twice or freed twice, under random
orders of requests; windows; slots.  The first cases are those of the reference's own
PagePool tests (crates/forward/src/core/scratch.rs:705-816)."""
import random

import pytest

from flambeau_amd.cache import CacheError, CacheManager, GroupSpec, PagePool


def mk(n_pages=8, page=4, slots=3, max_len=64, windows=(0,)):
    return CacheManager([GroupSpec(2, 8, w) for w in windows], n_pages, page, slots, max_len)


def test_pool_basics():
    p = PagePool(3)
    assert p.n_free == 3
    got = [p.acquire() for _ in range(3)]
    assert sorted(got) == [0, 1, 2] and p.acquire() is None and p.n_free == 0
    p.release(got[1])
    assert p.n_free == 1 and p.acquire() == got[1]
    p.release(got[0])
    with pytest.raises(CacheError, match="freed twice"):
        p.release(got[0])
    with pytest.raises(CacheError, match="not in the pool"):
        p.release(7)


def test_ensure_acquires_only_what_is_missing_and_all_or_nothing():
    m = mk()
    assert m.admit("a") is not None
    m.ensure("a", 5)                       # 2 pages of 4
    assert len(m.table_row("a", 0)) == 2 and m.free_pages() == [6]
    m.ensure("a", 8)                       # still 2
    assert m.free_pages() == [6]
    m.ensure("a", 9)
    assert m.free_pages() == [5]
    assert m.pages_needed("a", 32) == [5] and m.can_cover([("a", 32)])
    assert not m.can_cover([("a", 33)])
    with pytest.raises(CacheError, match="needs 6 pages, 5 free"):
        m.ensure("a", 33)
    assert m.free_pages() == [5]           # nothing was taken by the failed call
    with pytest.raises(CacheError, match="exceed the maximum"):
        m.ensure("a", 65)
    m.check_invariants()


def test_release_returns_everything_and_slots_are_reused():
    m = mk(slots=2)
    a, b = m.admit("a"), m.admit("b")
    assert {a.slot, b.slot} == {0, 1} and m.admit("c") is None
    assert sorted(m.take_fresh_slots()) == [0, 1] and m.take_fresh_slots() == []
    m.ensure("a", 16)
    m.ensure("b", 16)
    assert m.free_pages() == [0]
    m.release("a")
    assert m.free_pages() == [4] and m.n_free_slots == 1
    c = m.admit("c")
    assert c.slot == a.slot and m.take_fresh_slots() == [a.slot]
    with pytest.raises(CacheError, match="not live"):
        m.release("a")
    with pytest.raises(CacheError, match="already live"):
        m.admit("b")
    m.check_invariants()


def test_advance_beyond_pages_is_refused():
    m = mk()
    m.admit("a")
    m.ensure("a", 4)
    with pytest.raises(CacheError, match="beyond its pages"):
        m.advance("a", 5)


def test_window_gives_back_pages_that_all_future_queries_have_passed():
    m = mk(n_pages=6, page=4, windows=(6,), max_len=200)
    m.admit("a")
    m.ensure("a", 10)
    m.advance("a", 10)
    # next query at 10 sees keys >= 10 - 6 + 1 = 5: block 0 (tokens 0..3) is dead, block 1 (4..7) lives
    assert m.table_row("a", 0)[0] == -1 and m.table_row("a", 0)[1] >= 0 and m.free_pages() == [4]
    m.ensure("a", 12)
    m.advance("a", 2)
    # next query at 12 sees keys >= 7: block 1 still holds token 7
    assert m.table_row("a", 0)[1] >= 0
    m.ensure("a", 13)
    m.advance("a", 1)
    # next query at 13 sees keys >= 8: block 1 is dead now
    assert m.table_row("a", 0)[:2] == [-1, -1] and len(m.table_row("a", 0)) == 4
    m.check_invariants()
    # a long request never holds more than window/page + 2 pages
    for _ in range(150):
        n = m.live["a"].n_cached
        m.ensure("a", n + 1)
        m.advance("a", 1)
        assert sum(p >= 0 for p in m.table_row("a", 0)) <= 6 // 4 + 2
        m.check_invariants()
    m.release("a")
    assert m.free_pages() == [6]


def test_groups_are_separate():
    m = mk(n_pages=5, page=4, windows=(0, 4))
    m.admit("a")
    m.ensure("a", 16)
    m.advance("a", 16)
    assert m.free_pages()[0] == 1 and m.free_pages()[1] == 4     # the windowed group kept block 3 only
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    windows = (0, 5) if seed % 2 else (0,)
    m = mk(n_pages=12, page=4, slots=4, max_len=40, windows=windows)
    next_id = 0
    for _ in range(600):
        op = rng.random()
        live = list(m.live)
        if op < 0.25 and m.n_free_slots:
            m.admit(next_id)
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(live)
            k = rng.randint(1, 9)
            upto = m.live[rid].n_cached + k
            if m.can_cover([(rid, upto)]):
                m.ensure(rid, upto)
                m.advance(rid, k)
            else:
                with pytest.raises(CacheError):
                    m.ensure(rid, upto)
        elif live:
            m.release(rng.choice(live))
        m.check_invariants()
        for rc in m.live.values():
            for g, spec in enumerate(m.groups):
                # every key a future query needs has a page
                lo = max(0, rc.n_cached - spec.window + 1) if spec.window else 0
                for t in range(lo, rc.n_cached):
                    assert rc.tables[g][t // 4] >= 0
    for rid in list(m.live):
        m.release(rid)
    assert m.free_pages() == [12] * len(windows) and m.n_free_slots == 4
