"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of
requests; window groups give pages back; slots; block tables."""
import random

import numpy as np
import pytest

from gibbs_amd.cache import NO_PAGE, CacheManager, CacheNeed, PageError, PagePool, StateNeed

FULL = CacheNeed(2, 16)
WIN = CacheNeed(2, 16, window=40)


def manager(needs=(None, FULL, None, FULL), pages=12, reqs=3, ps=16):
    states = [(StateNeed("conv", (2, 8)),) if n is None else () for n in needs]
    return CacheManager(list(needs), states, ps, pages, reqs)


def test_pool_basics():
    p = PagePool(4)
    a = p.allocate(3)
    assert len(set(a)) == 3 and p.n_free == 1 and p.allocate(2) is None and p.n_free == 1
    p.release(a[:1])
    with pytest.raises(PageError, match="freed twice"):
        p.release(a[:1])
    with pytest.raises(PageError, match="not of this pool"):
        p.release([9])
    # a page that was just given back is the next one used
    assert p.allocate(1) == a[:1]


def test_groups_and_state_layout():
    m = manager(needs=(None, FULL, WIN, FULL, None, WIN))
    assert m.group_needs == [FULL, WIN] and m.group_layers == [[1, 3], [2, 5]]
    assert m.state_layout == {(0, "conv"): (0, (2, 8)), (4, "conv"): (16, (2, 8))} and m.slot_floats == 32


def test_reserve_commit_release():
    m = manager()
    assert m.admit("a") and m.admit("b")
    assert m.reserve("a", 17) and m.free_pages() == 10          # 17 tokens: 2 pages
    assert m.reserve("a", 17) and m.free_pages() == 10          # asking again takes nothing
    m.commit("a", 17)
    assert m.tokens("a") == 17 and m.pages_needed("a", 15) == [0] and m.pages_needed("a", 16) == [1]
    assert not m.reserve("b", 16 * 10 + 1) and m.free_pages() == 10, "a refused reservation takes nothing"
    assert m.reserve("b", 160) and m.free_pages() == 0
    with pytest.raises(PageError, match="beyond its reserved pages"):
        m.commit("a", 16)
    t = m.block_table(["b", "a"], 0)
    assert t.shape == (2, 10) and (t[0] >= 0).all() and (t[1, 2:] == NO_PAGE).all() and t.dtype == np.int32
    assert len(set(t[t >= 0].tolist())) == 12
    m.check()
    m.release("b")
    assert m.free_pages() == 10 and m.free_slots() == 2
    with pytest.raises(KeyError):
        m.release("b")
    m.check()


def test_slots_and_fresh():
    m = manager(reqs=2)
    assert m.admit(1) and m.admit(2) and not m.admit(3)
    assert sorted(m.take_fresh_slots()) == [0, 1] and m.take_fresh_slots() == []
    s = m.slot(1)
    m.release(1)
    assert m.admit(3) and m.slot(3) == s and m.take_fresh_slots() == [s], "a slot taken again is cleared again"
    with pytest.raises(KeyError):
        m.admit(3)


def test_window_group_returns_passed_pages():
    m = CacheManager([WIN, FULL], [(), ()], 16, 20, 2)
    m.admit("a")
    held = []
    for n in [30, 1, 1, 20, 50, 1]:
        assert m.reserve("a", n)
        m.commit("a", n)
        tokens = m.tokens("a")
        table = m.block_table(["a"], 0)[0]
        first_visible = max(0, tokens - 40 + 1)
        for j, p in enumerate(table):
            if (j + 1) * 16 <= first_visible:
                assert p == NO_PAGE, f"page {j} is behind the window at {tokens} tokens"
            elif j * 16 < tokens:
                assert p != NO_PAGE, f"page {j} holds visible keys at {tokens} tokens"
        held.append(20 - m.free_pages(0))
        m.check()
    assert max(held) <= 40 // 16 + 2 + 50 // 16, "a window group holds about a window of pages"
    assert 20 - m.free_pages(1) == m.pages_for(103), "the full group keeps every page"
    m.release("a")
    assert m.free_pages(0) == m.free_pages(1) == 20


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_invariants(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN, None], [(), (), (StateNeed("s", (3,)),)], 8, 30, 4)
    live, counter = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.free_slots():
            counter += 1
            assert m.admit(counter)
            live[counter] = 0
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 8, 9, 40])
            before = (m.free_pages(0), m.free_pages(1))
            if m.reserve(rid, n):
                m.commit(rid, n)
                live[rid] += n
                assert m.tokens(rid) == live[rid]
            else:
                assert (m.free_pages(0), m.free_pages(1)) == before
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        assert sorted(m.live()) == sorted(live)
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages(0) == m.free_pages(1) == 30 and m.free_slots() == 4
