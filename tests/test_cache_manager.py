"""The cache manager without a GPU: no page lost, held twice or freed twice, under random orders of requests;
groups with different needs; windows that give pages back; state slots."""
import random

import numpy as np
import pytest

from llm_infrence_engine_amd.cache import NULL_PAGE, CacheLayout, CacheManager, OutOfPages, PageAllocator
from llm_infrence_engine_amd.parts.base import KVNeed, StateNeed


def test_allocator_vectors_of_the_reference():
    """tests/test_paged.py:18-36 of the reference: 5 blocks give 1..4, never 0, a fifth raises; double free raises."""
    a = PageAllocator(4)
    got = [a.allocate() for _ in range(4)]
    assert sorted(got) == [1, 2, 3, 4] and NULL_PAGE not in got
    with pytest.raises(OutOfPages):
        a.allocate()
    for p in got:
        a.decref(p)
    assert a.num_free() == 4 and a.num_in_use() == 0
    a.check_invariants()
    p = a.allocate()
    a.decref(p)
    with pytest.raises(ValueError):
        a.decref(p)
    with pytest.raises(ValueError):
        a.decref(NULL_PAGE)


def test_shared_page_survives_until_the_last_holder_lets_go():
    a = PageAllocator(3)
    p = a.allocate()
    a.incref(p)
    a.decref(p)
    assert a.ref[p] == 1 and a.num_free() == 2
    a.decref(p)
    assert a.num_free() == 3
    with pytest.raises(ValueError):
        a.incref(p)
    a.check_invariants()


def test_freed_pages_are_used_again_in_order():
    a = PageAllocator(3)
    x, y, z = a.allocate(), a.allocate(), a.allocate()
    a.decref(y); a.decref(x)
    assert [a.allocate(), a.allocate()] == [y, x]


def full(nkv=2, d=16, window=None):
    return (KVNeed(nkv, d, window), None, None)


def test_layout_groups_runs_by_their_needs():
    needs = [full(), full(window=8), full(), (KVNeed(2, 16), None, 0), (None, StateNeed((4, 3)), None), full(4, 32)]
    lay = CacheLayout(needs)
    assert len(lay.group_keys) == 3
    assert lay.group_runs == [[0, 2], [1], [5]]
    assert lay.run_group == [0, 1, 0, 0, None, 2] and lay.run_entry == [0, 0, 1, 0, None, 0]
    assert lay.run_stores == [True, True, True, False, False, True]
    assert lay.state_runs == [4]
    with pytest.raises(ValueError, match="hold different tensors"):
        CacheLayout([full(), (KVNeed(4, 16), None, 0)])
    with pytest.raises(ValueError, match="further back"):
        CacheLayout([full(window=8), (KVNeed(2, 16), None, 0)])


def test_grow_advance_free():
    m = CacheManager(CacheLayout([full(), full()]), page_size=4, num_pages=10, max_requests=3, max_len=32)
    row = m.add("a")
    assert m.pages_to_grow("a", 9) == [3] and m.can_grow("a", 9) and not m.can_grow("a", 33)
    m.grow("a", 9)
    assert m.pages_held("a") == [[1, 2, 3]] and list(m.groups[0].tables[row, :4]) == [1, 2, 3, 0]
    m.grow("a", 9)                                  # nothing more to do
    assert m.num_free_pages() == [7]
    with pytest.raises(ValueError, match="allocated"):
        m.advance("a", 13)
    m.advance("a", 9)
    m.grow("a", 13)
    assert m.pages_held("a") == [[1, 2, 3, 4]]
    m.add("b")
    with pytest.raises(OutOfPages):
        m.grow("b", 4 * 7)                          # 7 pages wanted, 6 free: nothing is taken
    assert m.num_free_pages() == [6] and m.pages_held("b") == [[]]
    with pytest.raises(ValueError, match="made for"):
        m.grow("b", 33)
    m.free("a")
    assert m.num_free_pages() == [10] and not m.has("a")
    m.grow("b", 8)
    assert m.pages_held("b") == [[5, 6]]            # fresh pages first, freed ones go to the end of the line
    with pytest.raises(ValueError, match="already"):
        m.add("b")
    m.add("c"); m.add("d")
    with pytest.raises(OutOfPages, match="rows"):
        m.add("e")
    m.check_invariants()
    assert m.bytes_per_token(2) == 2 * 2 * 2 * 16 * 2


def test_window_gives_pages_back_once_passed():
    m = CacheManager(CacheLayout([full(), full(window=6)]), page_size=4, num_pages=8, max_requests=2, max_len=32)
    m.add("a")
    m.grow("a", 17)                                  # 5 pages in both groups
    assert m.num_free_pages() == [3, 3]
    m.advance("a", 17)                               # next query at 17 sees keys 12..17: pages 0..2 are passed
    assert m.pages_held("a")[0] == [1, 2, 3, 4, 5] and m.pages_held("a")[1] == [4, 5]
    assert list(m.groups[1].tables[m.row("a"), :5]) == [0, 0, 0, 4, 5]
    assert m.num_free_pages() == [3, 6]
    m.check_invariants()
    m.grow("a", 21)
    m.advance("a", 21)
    assert m.pages_held("a")[1] == [5, 6]            # page 4 was passed too
    m.add("b")
    m.grow("b", 8)
    assert m.pages_held("b") == [[7, 8], [7, 8]]
    m.free("b")
    m.free("a")
    assert m.num_free_pages() == [8, 8]
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    window = rng.choice([None, 5, 12])
    m = CacheManager(CacheLayout([full(), full(2, 16, window), full()]), page_size=rng.choice([1, 4, 16]),
                     num_pages=rng.choice([6, 20]), max_requests=4, max_len=96)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.free_rows():
            m.add(next_id); live[next_id] = 0; next_id += 1
        elif op < 0.8 and live:
            r = rng.choice(list(live))
            new = min(96, live[r] + rng.choice([1, 1, 1, 2, 7, 30]))
            if new > live[r] and m.can_grow(r, new):
                m.grow(r, new); m.advance(r, new); live[r] = new
            elif new > live[r]:
                before = m.num_free_pages()
                with pytest.raises(OutOfPages):
                    m.grow(r, new)
                assert m.num_free_pages() == before
        elif live:
            r = rng.choice(list(live))
            m.free(r); del live[r]
        m.check_invariants()
        for r, n in live.items():
            assert m.computed(r) == n
    for r in list(live):
        m.free(r)
    m.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in m.groups) and m.free_rows() == 4
    assert all((g.tables == NULL_PAGE).all() for g in m.groups)


def test_a_copy_kept_by_the_changed_entries_equals_the_tables():
    """What ``take_updates`` lists (each entry once per call) keeps a second copy of the block tables, the one the
    device holds, equal to the manager's, under random adds, growth, windows passing and frees; the last row
    stays all null pages."""
    rng = random.Random(5)
    m = CacheManager(CacheLayout([full(), full(window=6), full(4, 32)]), page_size=4, num_pages=[40, 12, 25],
                     max_requests=5, max_len=64)
    assert m.pages_per_group == [40, 12, 25] and m.num_pages == 12 and m.capacity_tokens() == 48
    copies = [np.zeros_like(g.tables) for g in m.groups]
    live, next_id = {}, 0
    for step in range(600):
        op = rng.random()
        if op < 0.25 and m.free_rows():
            m.add(next_id); live[next_id] = 0; next_id += 1
        elif op < 0.8 and live:
            r = rng.choice(list(live))
            n = min(64, live[r] + rng.randint(1, 9))
            if m.can_grow(r, n):
                m.grow(r, n); m.advance(r, n); live[r] = n
        elif live:
            r = rng.choice(list(live)); m.free(r); del live[r]
        if rng.random() < 0.4:                       # several operations between two steps is the usual case
            assert m.pending_updates() == max(len(c) for c in m._changed)
            for copy, (index, value) in zip(copies, m.take_updates()):
                assert len(set(index.tolist())) == index.size
                copy.reshape(-1)[index] = value
            assert m.pending_updates() == 0
            for copy, g in zip(copies, m.groups):
                assert (copy == g.tables).all() and (copy[m.null_row] == NULL_PAGE).all()
            m.check_invariants()


def test_tokens_that_fit_counts_every_group():
    m = CacheManager(CacheLayout([full(), full(4, 32)]), page_size=4, num_pages=[10, 3], max_requests=2, max_len=64)
    m.add("a")
    assert m.tokens_that_fit("a") == 12 and m.tokens_that_fit("a", reserve=1) == 8
    m.grow("a", 5); m.advance("a", 5)
    assert m.tokens_that_fit("a") == 7          # two pages held (8 tokens) and one free in the small pool, 5 stored
    with pytest.raises(ValueError, match="pool sizes"):
        CacheManager(CacheLayout([full()]), 4, [3, 3], 2, 64)
