"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of
requests; window groups give pages back; slots; block tables."""
import random

import numpy as np
import pytest

from gibbs_amd.cache import NO_PAGE, CacheManager, CacheNeed, PageError, StateNeed, host

FULL = CacheNeed(2, 16)
WIN = CacheNeed(2, 16, window=40)


def manager(needs=(None, FULL, None, FULL), pages=12, reqs=3, ps=16):
    states = [(StateNeed("conv", (2, 8)),) if n is None else () for n in needs]
    return CacheManager(list(needs), states, ps, pages, reqs)


class PagePool:
    """A handle on one pool of the native core (the cache manager holds one per group)."""

    def __init__(self, num_pages: int):
        self.lib, self.num_pages = host.library(), num_pages
        self.pool = self.lib.gibbs_pool_create(num_pages)

    def __del__(self):
        self.lib.gibbs_pool_destroy(self.pool)

    @property
    def n_free(self) -> int:
        return self.lib.gibbs_pool_free(self.pool)

    def allocate(self, n: int):
        out = host.ints([0] * n)
        return None if self.lib.gibbs_pool_allocate(self.pool, n, out) < 0 else list(out[:n])

    def release(self, pages) -> None:
        pages = list(pages)
        if self.lib.gibbs_pool_release(self.pool, host.ints(pages), len(pages)) < 0:
            raise PageError(host.last_error())


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
    assert m.state_layout == {(0, "conv"): (0, (2, 8), "float32"), (4, "conv"): (16, (2, 8), "float32")} and m.slot_floats == 32
    typed = CacheManager([None], [(StateNeed("a", (3,), "bfloat16"), StateNeed("n", (1,), "int32"), StateNeed("b", (2, 2)))], 8, 4, 2)
    assert typed.state_layout == {(0, "a"): (0, (3,), "bfloat16"), (0, "n"): (2, (1,), "int32"), (0, "b"): (3, (2, 2), "float32")}
    assert typed.slot_floats == 7
    with pytest.raises(ValueError, match="float64"):
        StateNeed("x", (1,), "float64")


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


def test_reserve_and_commit_for_several_requests_at_once():
    """What a decode loop asks before and after its steps: pages for the next positions of all its requests, all or
    nothing, and the commit of all of them, each in one call of the core."""
    m = manager()                                                # 12 pages of 16 tokens
    for r in "abc":
        assert m.admit(r)
    assert m.reserve("a", 30) and m.reserve("b", 16) and m.reserve("c", 5)
    m.commit("a", 30); m.commit("b", 16); m.commit("c", 5)
    assert m.free_pages() == 8
    assert m.reserve_all(["a", "b", "c"], 2) is True and m.pages_needed_all == [1], "only b stands at a page's edge"
    assert m.free_pages() == 7
    assert m.reserve_all(["a", "b", "c"], 2) is False and m.free_pages() == 7, "asking again takes nothing"
    m.commit_all(["a", "b", "c"], 2)
    assert [m.tokens(r) for r in "abc"] == [32, 18, 7]
    assert m.reserve_all(["a", "b", "c"], 16 * 3) is None and m.pages_needed_all == [9] and m.free_pages() == 7, \
        "3 + 3 + 3 pages do not fit 7: nothing is taken"
    assert m.reserve_all(["a", "b"], 16 * 3) is True and m.free_pages() == 1
    with pytest.raises(ValueError, match="context limit"):
        m.reserve_all(["c"], 10, limit=16)
    with pytest.raises(PageError, match="beyond its reserved pages"):
        m.commit_all(["a", "c"], 48)
    assert m.tokens("a") == 32, "a commit that one request cannot take changes none"
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


def test_groups_with_pools_of_their_own_size():
    """A group with a window does with a pool much smaller than the group that keeps every key; keys and
    values with different head sizes are a need of their own."""
    m = CacheManager([FULL, WIN, FULL], [(), (), ()], 16, [40, 6], 2)
    assert [p.num_pages for p in m.pools] == [40, 6] and m.group_layers == [[0, 2], [1]]
    m.admit("a")
    for n in [30, 20, 1, 40, 40, 1, 33]:          # 165 tokens: 11 pages of the full group, never more than 6 of the window's
        assert m.reserve("a", n), f"the window group ran out at {m.tokens('a')} + {n} tokens"
        assert m.free_pages(1) >= 0
        m.commit("a", n)
        m.check()
    assert 40 - m.free_pages(0) == m.pages_for(165) and 6 - m.free_pages(1) <= 40 // 16 + 2
    assert not m.reserve("a", 16 * 5), "a portion that the small pool cannot hold beside the window is refused"
    assert m.free_pages(1) == 6 - (m.pages_for(165) - (165 - 40 + 1) // 16) and m.tokens("a") == 165
    m.release("a")
    assert (m.free_pages(0), m.free_pages(1)) == (40, 6)
    with pytest.raises(ValueError, match="page counts"):
        CacheManager([FULL, WIN], [(), ()], 16, [40], 2)
    wide_values = CacheNeed(2, 16, v_head_dim=24)
    assert wide_values != FULL and wide_values.value_dim == 24 and FULL.value_dim == 16
    m = CacheManager([FULL, wide_values, FULL], [(), (), ()], 16, 8, 2)
    assert m.group_needs == [FULL, wide_values] and m.group_layers == [[0, 2], [1]]


def test_a_slot_given_back_before_any_step_is_listed_once():
    """Admission that is undone (the scheduler tries the head of its queue and finds no room) must not
    pile the slot up among the fresh ones: every fresh slot is reported, each once."""
    m = manager(reqs=3)
    for i in range(10):
        assert m.admit(("try", i))
        m.release(("try", i))
    assert m.admit("a") and m.admit("b") and m.admit("c")
    assert sorted(m.take_fresh_slots()) == [0, 1, 2] and m.take_fresh_slots() == []


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


def test_native_step_staging_matches_a_plain_packing():
    """The host runtime's packing of a step (ids, positions, row -> request, cu, ctx, slots, wanted rows,
    block tables, every section on a 16-byte boundary) against the same arrays built here; a refused
    step (bad token, wanted place, context limit, too few pages) changes nothing."""
    import ctypes

    from gibbs_amd.cache import host
    lib = host.library()
    m = CacheManager([FULL, None, WIN], [(), (StateNeed("s", (4,)),), ()], 8, 10, 4)
    rng = random.Random(3)
    for rid, n in (("a", 11), ("b", 3)):
        assert m.admit(rid) and m.reserve(rid, n)
        m.commit(rid, n)
    assert m.admit("c")

    def stage(entries, vocab=100, ctx_limit=64):
        n = len(entries)
        slots = np.array([m.slot(r) for r, _, _ in entries], dtype=np.int32)
        q_len = np.array([len(t) for _, t, _ in entries], dtype=np.int32)
        tokens = np.array([x for _, t, _ in entries for x in t], dtype=np.int32)
        want_cu = np.concatenate([[0], np.cumsum([len(w) for _, _, w in entries])]).astype(np.int32)
        want = np.array([x for _, _, w in entries for x in w], dtype=np.int32)
        info = (ctypes.c_long * (1 + m.n_groups))()
        bad = ctypes.c_int(-1)
        ops = (n, slots.ctypes.data, q_len.ctypes.data, tokens.ctypes.data, want_cu.ctypes.data, want.ctypes.data)
        code = lib.gibbs_cache_reserve_step(m.core, *ops, vocab, ctx_limit, info, ctypes.byref(bad))
        if code < 0:
            return code, bad.value, host.last_error()
        out = np.full(int(info[0]), -7, dtype=np.int32)
        offsets = (ctypes.c_long * (9 + m.n_groups))()
        assert lib.gibbs_cache_fill_step(m.core, *ops, info, out.ctypes.data, offsets) == 0
        return out, list(offsets), [int(info[1 + g]) for g in range(m.n_groups)]

    before = (m.free_pages(0), m.free_pages(1))
    assert stage([("a", [1, 2], [0]), ("b", [3, 100], [])])[:2] == (host.ERR_STEP, 1)          # token outside the vocabulary
    assert stage([("a", [1, 2], [2])])[:2] == (host.ERR_STEP, 0)                                # wanted place outside
    assert stage([("a", [1] * 54, [])])[0] == host.ERR_STEP                                     # 65 tokens > 64
    assert stage([("a", [1], []), ("a", [2], [])])[:2] == (host.ERR_STEP, 1)                    # twice in one step
    code, group, text = stage([("a", [1] * 30, []), ("c", [1] * 50, [])])
    assert code == host.ERR_NO_ROOM and "pages" in text
    assert (m.free_pages(0), m.free_pages(1)) == before and m.tokens("a") == 11
    m.check()

    entries = [("b", [7], [0]), ("a", [rng.randrange(100) for _ in range(9)], [0, 8]), ("c", [5, 6, 7], [])]
    out, offsets, widths = stage(entries)
    ctx = [3, 11, 0]
    q = [1, 9, 3]
    cu = np.concatenate([[0], np.cumsum(q)])
    assert all(o % 4 == 0 for o in offsets[:7 + m.n_groups])
    sec = lambda i, size: out[offsets[i]:offsets[i] + size].tolist()
    assert sec(0, 13) == [x for _, t, _ in entries for x in t]
    assert sec(1, 13) == [c + t for c, n in zip(ctx, q) for t in range(n)]
    assert sec(2, 13) == [i for i, n in enumerate(q) for _ in range(n)]
    assert sec(3, 4) == cu.tolist() and sec(4, 3) == ctx and sec(5, 3) == [m.slot(r) for r, _, _ in entries]
    assert sec(6, 3) == [0, 1, 9]                                                               # b's row, rows of a's places 0 and 8
    for g in range(m.n_groups):
        table = np.array(sec(7 + g, 3 * widths[g])).reshape(3, widths[g])
        assert (table == m.block_table([r for r, _, _ in entries], g, widths[g])).all()
        assert widths[g] == m.pages_for(20)
    assert offsets[7 + m.n_groups:9 + m.n_groups] == [9, 20]                                     # longest portion, longest sequence
    for (r, t, _), n in zip(entries, q):
        m.commit(r, n)
    m.check()
