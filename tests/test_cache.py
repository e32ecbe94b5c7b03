"""The cache's bookkeeping: slots, pages, windows (CPU, no storage)."""
import random

import numpy as np
import pytest

from sonicboom_amd.cache import CacheError, GroupSpec, PagedCache, PagePool, group_entries, pages_for


def make(max_tokens=64 * 8, window=0, max_slots=None):
    groups = [GroupSpec(2, 16, 0, (0, 1))]
    if window:
        groups.append(GroupSpec(1, 32, window, (2,)))
    return PagedCache(groups, max_tokens, allocate=False, max_slots=max_slots)


def check_invariants(c: PagedCache):
    """No page lost or held twice: every page is either free or in exactly one slot's list."""
    for g, pool in enumerate(c.pools):
        held = [p for s in c.live_slots for p in c._slots[s].pages[g] if p >= 0]
        assert len(held) == len(set(held)), "a page is held twice"
        assert len(held) + pool.free_count == pool.n_pages, "a page is lost"
        assert set(held).isdisjoint(pool._free)
    assert len(c.live_slots) + len(c._free_slots) == c.max_slots
    assert set(c.live_slots).isdisjoint(c._free_slots)


def test_page_pool_refuses_double_free():
    p = PagePool(3)
    a, b = p.alloc(), p.alloc()
    p.free(a)
    with pytest.raises(CacheError):
        p.free(a)
    with pytest.raises(CacheError):
        p.free(7)
    p.alloc(), p.alloc()
    with pytest.raises(CacheError, match="out of cache pages"):
        p.alloc()


def test_slots_are_given_back_and_used_again():
    c = make(max_slots=2)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(CacheError, match="out of sequence slots"):
        c.alloc_slot()
    c.reserve([a, b], [70, 1])
    c.advance([a, b], [70, 1])
    assert (c.length(a), c.length(b)) == (70, 1) and c.held_pages() == 3
    c.free_slot(a)
    with pytest.raises(CacheError, match="freed while not in use"):
        c.free_slot(a)
    with pytest.raises(CacheError, match="not in use"):
        c.length(a)
    assert c.held_pages() == 1
    a2 = c.alloc_slot()
    assert a2 == a and c.length(a2) == 0       # the same slot again, empty
    check_invariants(c)


def test_max_tokens_counts_each_sequence_rounded_up_to_a_page():
    c = make(max_tokens=64 * 3)
    s = [c.alloc_slot() for _ in range(3)]
    c.reserve(s, [1, 64, 5])                  # 1 + 1 + 1 pages
    c.advance(s, [1, 64, 5])
    with pytest.raises(CacheError, match="out of cache pages"):
        c.reserve([s[1]], [1])                # position 64 needs a second page
    c.reserve([s[0]], [63])                   # still inside its first page
    c.advance([s[0]], [63])
    check_invariants(c)


def test_reserve_is_all_or_nothing():
    c = make(max_tokens=64 * 4)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(CacheError):
        c.reserve([a, b], [128, 200])         # 2 + 4 pages > 4
    assert c.held_pages() == 0
    with pytest.raises(CacheError, match="twice"):
        c.reserve([a, a], [1, 1])
    with pytest.raises(CacheError, match="at least one token"):
        c.reserve([a], [0])
    check_invariants(c)


def test_page_table_maps_positions_to_pages():
    c = make()
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a, b], [130, 3])
    t = c.page_table(0, [b, a])
    assert t.dtype == np.int32 and t.shape == (2, 3)
    assert (t[0, 1:] == -1).all() and (t[1] >= 0).all() and len(set(t[1]) | {t[0, 0]}) == 4


def test_windowed_group_gives_pages_back():
    c = make(max_tokens=64 * 16, window=100)
    s = c.alloc_slot()
    c.reserve([s], [300])
    assert c.held_pages(0) == 5 and c.held_pages(1) == 5      # a long prompt needs all its pages in the step
    c.advance([s], [300])
    # next query at 300 reads keys 201..300: pages 3.. stay, 0..2 go back
    assert c.held_pages(0) == 5 and c.held_pages(1) == 2
    t = c.page_table(1, [s])
    assert (t[0, :3] == -1).all() and (t[0, 3:5] >= 0).all()
    for _ in range(200):
        c.reserve([s], [1])
        c.advance([s], [1])
        assert c.held_pages(1) <= pages_for(100) + 1
    check_invariants(c)
    c.free_slot(s)
    assert c.held_pages(0) == 0 and c.held_pages(1) == 0


def test_random_traffic_keeps_the_books():
    rnd = random.Random(7)
    c = make(max_tokens=64 * 40, window=70, max_slots=6)
    live = {}
    for _ in range(600):
        r = rnd.random()
        if r < 0.25 and len(live) < 6:
            live[c.alloc_slot()] = 0
        elif r < 0.4 and live:
            s = rnd.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            chosen = rnd.sample(list(live), rnd.randint(1, len(live)))
            n = [rnd.choice([1, 1, 1, 17, 64, 90]) for _ in chosen]
            try:
                c.reserve(chosen, n)
            except CacheError:
                check_invariants(c)
                continue
            c.advance(chosen, n)
            for s, k in zip(chosen, n):
                live[s] += k
        check_invariants(c)
        assert all(c.length(s) == n for s, n in live.items())


def test_groups_by_need():
    g = group_entries({0: (2, 16, 0), 1: (2, 16, 0), 2: (2, 16, 128), 3: (4, 16, 0)})
    assert [(x.kv_heads, x.head_dim, x.window, x.entries) for x in g] == [
        (2, 16, 0, (0, 1)), (2, 16, 128, (2,)), (4, 16, 0, (3,))]
    with pytest.raises(CacheError, match="two groups"):
        PagedCache([GroupSpec(1, 16, 0, (0,)), GroupSpec(1, 16, 4, (0,))], 64, allocate=False)


def test_groups_of_rows_beside_keys_and_values():
    """Entries that keep a row of their own shape per token form groups by (shape, window), apart
    from the groups of keys and values; their pages are counted and given back like the others'."""
    g = group_entries({0: ("rows", (12,), 0), 1: (1, 16, 0), 2: ("rows", (12,), 0), 3: ("rows", (12,), 70),
                       4: ("rows", (3, 4), 0)})
    assert [(x.row_shape, x.kv_heads, x.head_dim, x.window, x.entries) for x in g] == [
        ((12,), 0, 0, 0, (0, 2)), ((), 1, 16, 0, (1,)), ((12,), 0, 0, 70, (3,)), ((3, 4), 0, 0, 0, (4,))]
    c = PagedCache(g, 64 * 6, allocate=False)
    s = c.alloc_slot()
    c.reserve([s], [200])
    c.advance([s], [200])
    assert [c.held_pages(i) for i in range(4)] == [4, 4, 2, 4]      # the window of 70 has let two pages go
    c.free_slot(s)
    assert [c.held_pages(i) for i in range(4)] == [0, 0, 0, 0]


def test_the_caches_order_of_elements_is_a_permutation_of_every_row():
    """cache.layout (the Python face of sb_key_index / sb_value_index): within a row the groups
    of eight elements are permuted, nothing is lost or doubled, elements keep their place within
    a group, head sizes that are no multiple of 16 keep the plain order, and the sixteen keys that
    a matrix-core fragment read touches at once get sixteen different group offsets when the row
    has that many groups."""
    from sonicboom_amd.cache import layout
    for hd in (8, 16, 24, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 240, 256):
        kp, vp = layout.key_positions(hd), layout.value_positions(hd)
        assert kp.shape == (64, hd) and vp.shape == (hd, 64)
        for j in range(64):
            assert sorted(kp[j].tolist()) == list(range(hd))
            assert (kp[j] % 8 == np.arange(hd) % 8).all()
        for d in range(hd):
            assert sorted(vp[d].tolist()) == list(range(64))
            assert (vp[d] % 8 == np.arange(64) % 8).all()
        if hd % 16:
            assert (kp == np.arange(hd)[None, :]).all()
    kp = layout.key_positions(128)
    keys = [8 * a + i for a in range(4) for i in range(4)]                      # one score tile's rows
    assert len({int(kp[j, 0]) // 8 for j in keys}) == 16
    vp = layout.value_positions(128)
    assert len({(int(vp[d, 0]) // 8, d % 2) for d in range(16)}) == 16           # sixteen rows: 8 offsets x 2 rows of 128 bytes


def test_a_windowed_group_gets_a_pool_of_its_own_size():
    """With bounds on the sequences and on the rows between two advances, a windowed group holds
    at most a window and a step's rows a sequence: its pool is that big and never runs out,
    whatever the lengths; the group that keeps every key is what refuses."""
    from sonicboom_amd.cache.paged import pool_pages
    assert pool_pages(100, 0, 4, 64) == 100 and pool_pages(100, 50, 4, 0) == 100
    assert pool_pages(100, 50, 4, 64) == 4 * 3 + 1 and pool_pages(10, 50, 4, 64) == 10
    groups = [GroupSpec(2, 16, 0, (0,)), GroupSpec(1, 32, 100, (1,))]
    c = PagedCache(groups, 64 * 40, allocate=False, max_slots=3, step_rows=128)
    assert [p.n_pages for p in c.pools] == [40, 3 * 4 + 2]
    rng = random.Random(3)
    slots = [c.alloc_slot() for _ in range(3)]
    for _ in range(60):
        # a step of at most 128 rows over the three sequences, in any split
        total = rng.randint(3, 128)
        first = rng.randint(1, total - 2)
        second = rng.randint(1, total - first - 1)
        n_new = [first, second, total - first - second]
        try:
            c.reserve(slots, n_new, c.windowed(False))
        except CacheError:
            break                                   # the full group is out of pages: 40 pages are held
        c.reserve(slots, n_new, c.windowed(True))   # never refuses
        c.advance(slots, n_new)
        check_invariants(c)
        assert c.held_pages(1) <= 3 * 3
    else:
        raise AssertionError("the cache never filled up")
    assert c.windowed(True) == [1] and c.windowed(False) == [0]


def test_trim_gives_back_what_was_reserved_for_rows_that_did_not_run():
    c = make(window=70)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a, b], [100, 10])
    c.advance([a, b], [100, 10])
    before = [c.held_pages(g) for g in range(2)]
    c.reserve([a, b], [200, 60])                    # a step that then fails: nothing advances
    assert c.held_pages(0) == before[0] + 3 + 1
    c.trim([a, b])
    assert [c.held_pages(g) for g in range(2)] == before
    assert (c.length(a), c.length(b)) == (100, 10)
    check_invariants(c)
    c.trim([a])                                     # nothing to give back: no harm
    c.reserve([a], [1])
    c.advance([a], [1])
    check_invariants(c)
