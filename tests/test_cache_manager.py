"""The cache manager (no GPU): no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; state slots."""
import random

import pytest

from deliverance_amd.cache import CacheError, CacheManager, KVGroupSpec, OutOfPages, PagePool, StateSpec


def full(n_pages=8, page=4, slots=0):
    return CacheManager([KVGroupSpec((0, 1), 2, 16, None)], page, [n_pages],
                        [StateSpec(2, 5)] if slots else [], slots)


def test_pool_refuses_double_free_and_foreign_pages():
    p = PagePool(3)
    a = p.take(2, "a")
    assert a == [0, 1] and p.n_free == 1
    with pytest.raises(OutOfPages):
        p.take(2, "b")
    with pytest.raises(CacheError, match="belongs to"):
        p.give([a[0]], "b")
    p.give(a, "a")
    with pytest.raises(CacheError, match="freed twice"):
        p.give([a[0]], "a")
    assert p.n_free == 3


def test_block_table_grows_by_pages_and_addresses_rows():
    m = full()
    m.open("r")
    assert m.extend("r", 5) == 0            # positions 0..4 need two pages of 4
    assert len(m.table("r", 0)) == 2
    m.commit("r")
    assert m.length("r") == 5
    t = m.table("r", 0)
    # rows written at positions 0..4 are read back in order across pages
    # (the reference's round trip: core/src/test/java/io/teknek/deliverance/tensor/KvBufferCachePrefixTest.java:103-153)
    assert m.slots_for("r", 0, 0, 5) == [t[0] * 4 + 0, t[0] * 4 + 1, t[0] * 4 + 2, t[0] * 4 + 3, t[1] * 4 + 0]
    assert m.extend("r", 3) == 5            # fills page 2 exactly: no new page
    assert len(m.table("r", 0)) == 2
    m.commit("r")
    assert m.extend("r", 1) == 8 and len(m.table("r", 0)) == 3   # the page's edge
    m.commit("r")
    m.check()
    m.close("r")
    assert m.pools[0].n_free == 8
    m.check()


def test_extend_is_all_or_nothing_and_rollback_returns_pages():
    m = full(n_pages=3)
    m.open("a"); m.open("b")
    m.extend("a", 8); m.commit("a")
    with pytest.raises(OutOfPages):
        m.extend("b", 5)
    assert m.table("b", 0) == [] and m.pools[0].n_free == 1
    assert not m.can_extend("b", 5) and m.can_extend("b", 4)
    m.extend("b", 3)
    m.rollback("b")
    assert m.table("b", 0) == [] and m.pools[0].n_free == 1 and m.length("b") == 0
    m.check()


def test_unknown_and_duplicate_requests():
    m = full()
    with pytest.raises(CacheError, match="not open"):
        m.extend("x", 1)
    m.open("x")
    with pytest.raises(CacheError, match="already open"):
        m.open("x")
    m.close("x")
    with pytest.raises(CacheError, match="not open"):
        m.close("x")


def test_window_group_gives_pages_back_once_passed():
    # window 6, pages of 4: a query at position p sees keys p-5..p
    m = CacheManager([KVGroupSpec((0,), 1, 16, None), KVGroupSpec((1,), 1, 16, 6)], 4, [16, 16])
    m.open("r")
    m.extend("r", 9); released = m.commit("r")
    # next query sits at 9 and sees 4..9: page 0 (positions 0..3) is passed
    assert released == [(1, m.table("r", 1)[0])] or m.table("r", 1)[0] == -1
    assert m.table("r", 1)[0] == -1 and m.table("r", 1)[1] >= 0
    assert all(p >= 0 for p in m.table("r", 0))          # the full group keeps everything
    with pytest.raises(CacheError, match="given back"):
        m.slots_for("r", 1, 2, 1)
    for _ in range(20):
        m.extend("r", 1); m.commit("r"); m.check()
    live = [p for p in m.table("r", 1) if p >= 0]
    assert len(live) <= 3                                 # at most ceil(6/4)+1 pages stay
    assert m.pools[1].n_free == 16 - len(live)
    m.close("r")
    assert m.pools[1].n_free == 16 and m.pools[0].n_free == 16


def test_state_slots_are_handed_out_and_returned():
    m = full(slots=2)
    a, b = m.open("a"), m.open("b")
    assert {a, b} == {0, 1} and not m.can_open()
    with pytest.raises(OutOfPages):
        m.open("c")
    m.close("a")
    assert m.can_open() and m.open("c") == a
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_invariant(seed):
    rng = random.Random(seed)
    page = rng.choice([2, 4, 16])
    n_pages = rng.randint(6, 30)
    window = rng.choice([None, 5, 17])
    m = CacheManager([KVGroupSpec((0,), 2, 16, None), KVGroupSpec((1,), 2, 16, window)], page, [n_pages, n_pages],
                     [StateSpec(2, 3)], 4)
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.can_open():
            m.open(next_id); live[next_id] = 0; next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.randint(1, 3 * page)
            if m.can_extend(rid, n):
                start = m.extend(rid, n)
                assert start == live[rid]
                if rng.random() < 0.15:
                    m.rollback(rid)
                else:
                    m.commit(rid); live[rid] += n
            else:
                with pytest.raises(OutOfPages):
                    m.extend(rid, n)
        elif live:
            rid = rng.choice(list(live))
            m.close(rid); del live[rid]
        m.check()
        for rid, n in live.items():
            assert m.length(rid) == n
    for rid in list(live):
        m.close(rid)
    m.check()
    assert [p.n_free for p in m.pools] == [n_pages, n_pages]


def test_release_hook_sees_every_page_that_goes_back():
    """close, rollback and the window's release all report the pages they give back (a debug run
    fills them with NaN on the device)."""
    mgr = CacheManager([KVGroupSpec((0,), 1, 16, None), KVGroupSpec((1,), 1, 16, 20)], 16, [8, 8])
    seen = []
    mgr.on_release = lambda g, pages: seen.append((g, list(pages)))
    mgr.open("a")
    mgr.extend("a", 40)
    released = mgr.commit("a")                       # the window of 20 has passed page 0 of group 1
    assert seen == [(g, [p]) for g, p in released] and [g for g, _ in seen] == [1]
    seen.clear()
    mgr.extend("a", 30)
    before = {g: list(mgr.table("a", g)) for g in (0, 1)}
    mgr.rollback("a")
    after = {g: list(mgr.table("a", g)) for g in (0, 1)}
    assert sorted(p for g, ps in seen for p in ps if g == 0) == sorted(set(before[0]) - set(after[0]))
    seen.clear()
    held = {g: [p for p in mgr.table("a", g) if p >= 0] for g in (0, 1)}
    mgr.close("a")
    assert {g: ps for g, ps in seen} == held
    mgr.check()
    assert all(pool.n_free == 8 for pool in mgr.pools)
