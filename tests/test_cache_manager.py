"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; slots; prefix sharing (no GPU)."""
import random

import pytest

from ullm_amd.cache.manager import CacheFull, CacheGroupSpec, CacheManager
from ullm_amd.cache.pages import PageAllocator, PageError
from ullm_amd.cache.prefix_tree import PrefixTree

FULL = CacheGroupSpec(2, 16, 0, (0,))
WIN = CacheGroupSpec(2, 16, 10, (1, 2))


def test_allocator_all_or_nothing_and_double_free():
    a = PageAllocator(4)
    assert a.alloc(5) is None and a.num_free == 4
    pages = a.alloc(3)
    assert sorted(pages) == [0, 1, 2] and a.num_free == 1
    a.incref(pages[0])
    assert a.decref(pages[0]) is False and a.decref(pages[0]) is True
    with pytest.raises(PageError):
        a.decref(pages[0])
    with pytest.raises(PageError):
        a.incref(3)                      # never handed out
    a.check()
    # LIFO: the page just freed is handed out next (it is reused)
    assert a.alloc(1) == [pages[0]]


def test_reserve_commit_release_and_table_growth():
    m = CacheManager([FULL], [6], page_size=4, max_requests=2)
    rc = m.admit("a")
    assert m.pages_needed(rc, 1) == [1] and m.pages_needed(rc, 4) == [1] and m.pages_needed(rc, 5) == [2]
    assert m.reserve(rc, 5) and len(rc.tables[0]) == 2
    m.commit(rc, 5)
    assert rc.num_computed == 5 and m.pages_needed(rc, 3) == [0] and m.pages_needed(rc, 4) == [1]
    with pytest.raises(PageError):
        m.commit(rc, 4)                  # computed past what was reserved
    assert rc.num_computed == 5
    assert not m.reserve(rc, 4 * 5) and len(rc.tables[0]) == 2       # nothing taken on failure
    m.release(rc)
    assert m.num_free_pages() == 6 and m.num_free_slots == 2
    with pytest.raises(PageError):
        m.release(rc)
    m.check()


def test_slots_run_out_and_are_used_again():
    m = CacheManager([FULL], [4], page_size=4, max_requests=2)
    a, b = m.admit("a"), m.admit("b")
    assert {a.slot, b.slot} == {0, 1} and a.num_computed == 0
    with pytest.raises(CacheFull):
        m.admit("c")
    with pytest.raises(PageError):
        m.admit("a")
    m.release(a)
    c = m.admit("c")
    assert c.slot == a.slot and c.num_computed == 0      # a request that starts at 0 has its state rows zeroed by the step
    m.check()


def test_window_gives_pages_back_as_it_passes():
    m = CacheManager([FULL, WIN], [16, 16], page_size=4, max_requests=1)
    rc = m.admit("a")
    for step in range(40):
        assert m.reserve(rc, 1)
        m.commit(rc, 1)
        n = rc.num_computed
        held = [i for i, p in enumerate(rc.tables[1]) if p >= 0]
        # the next query (position n) reads keys n-9 .. n: their pages must be held, earlier ones not
        first_needed = max(0, n - 10 + 1) // 4
        assert held and held[0] == first_needed, (n, held)
        assert len(rc.pages_held(0)) == -(-n // 4)
        m.check()
    assert len(rc.pages_held(1)) <= 4
    m.release(rc)
    assert m.num_free_pages(0) == 16 and m.num_free_pages(1) == 16


def test_window_with_portions():
    m = CacheManager([WIN], [8], page_size=4, max_requests=1)
    rc = m.admit("a")
    assert m.reserve(rc, 19)            # a portion longer than the window needs all its pages during the step
    assert len(rc.pages_held(0)) == 5
    m.commit(rc, 19)                    # next query at 19 reads from 10: pages 0,1 (rows 0..7) are dead
    assert [p >= 0 for p in rc.tables[0]] == [False, False, True, True, True]
    m.check()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_conserve_pages(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN], [24, 12], page_size=4, max_requests=4, enable_prefix_cache=False)
    live = {}
    n_admitted = 0
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and m.num_free_slots:
            rid = f"r{n_admitted}"
            n_admitted += 1
            live[rid] = m.admit(rid)
        elif op < 0.85 and live:
            rc = live[rng.choice(sorted(live))]
            n = rng.choice([1, 1, 1, 2, 5, 9])
            before = [a.num_free for a in m.allocators]
            if m.reserve(rc, n):
                m.commit(rc, n)
            else:
                assert [a.num_free for a in m.allocators] == before
        elif live:
            rid = rng.choice(sorted(live))
            m.release(live.pop(rid))
        m.check()
        tables = [set(rc.pages_held(0)) for rc in live.values()]
        assert sum(len(t) for t in tables) == len(set().union(*tables)) if tables else True
    for rc in live.values():
        m.release(rc)
    m.check()
    assert m.num_free_pages(0) == 24 and m.num_free_pages(1) == 12 and m.num_free_slots == 4


def test_prefix_tree_vector_from_the_reference_comment():
    """ullm/core/kv_cache.py:370-377 at page size 1: seq1 [1,2,3,4] -> slots [10,11,12,13], seq2
    [1,2,3,5] -> [20,21,22,23]; afterwards the tree holds [1,2,3] -> [10,11,12], 4 -> 13, 5 -> 23 and the
    duplicates 20,21,22 are free once seq2 lets go."""
    alloc = PageAllocator(32)
    alloc.alloc(32)
    for p in range(32):
        if p not in (10, 11, 12, 13, 20, 21, 22, 23):
            alloc.decref(p)
    tree = PrefixTree(1, [alloc])
    assert tree.insert([1, 2, 3, 4], 4, [[10, 11, 12, 13]]) == 4
    assert tree.insert([1, 2, 3, 5], 4, [[20, 21, 22, 23]]) == 1
    for p in (10, 11, 12, 13, 20, 21, 22, 23):     # the requests let go
        alloc.decref(p)
    assert sorted(tree.pages_held(0)) == [10, 11, 12, 13, 23]
    assert all(alloc.refcount(p) == 0 for p in (20, 21, 22))
    got = tree.match([1, 2, 3, 5, 9], 4)
    assert [g[0] for g in got] == [10, 11, 12, 23]
    alloc.check()


def test_prefix_sharing_through_the_manager():
    m = CacheManager([FULL], [8], page_size=4, max_requests=3, enable_prefix_cache=True)
    prompt = list(range(100, 111))                        # 11 tokens: 2 full pages + 3
    a = m.admit("a", prompt)
    assert a.num_computed == 0
    assert m.reserve(a, 11)
    m.commit(a, 11)
    pages_a = list(a.tables[0])
    m.release(a, tokens=prompt)
    assert m.num_free_pages() == 6                        # two full pages stay with the tree
    b = m.admit("b", prompt[:9] + [7, 7])
    assert b.num_computed == 8 and b.tables[0] == pages_a[:2]
    c = m.admit("c", prompt[:8])                          # a match must leave one token to compute
    assert c.num_computed == 4
    m.check()
    # a one-token prompt (the reference's match_prefix fails on it, ullm/core/kv_cache.py:176-178,351)
    m.release(c)
    d = m.admit("d", [5])
    assert d.num_computed == 0
    # shared pages survive the release of one holder and are evicted only when nobody reads them
    assert m.reserve(b, 3)
    m.commit(b, 3)
    m.release(d)
    e = m.admit("e", [1, 2, 3])
    assert not m.reserve(e, 4 * 6)                        # b still reads the shared pages: not evictable
    m.release(b, tokens=prompt[:9] + [7, 7])
    assert m.reserve(e, 4 * 8)                            # now the tree's pages are evicted for e
    m.check()
    assert m.prefix_tree.num_nodes == 0


def test_prefix_sharing_is_off_with_windows():
    m = CacheManager([FULL, WIN], [8, 8], page_size=4, max_requests=2, enable_prefix_cache=True)
    assert m.prefix_tree is None
