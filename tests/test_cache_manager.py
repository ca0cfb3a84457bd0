"""The allocator and the cache manager: no page lost, held twice or freed twice, under random
orders of requests; windows give pages back; slots."""

import random

import pytest

from from_scratch_inference_engine_amd.cache import (CacheManager, NoFreeSlot, OutOfPages, PageAllocator,
                                                     PagedNeed)


def test_allocator_semantics():
    # tests/cpp/test_block_allocator.cpp: distinct ids from 0, throw when empty, freed id reused
    # next, a reference count delays the free, double free throws
    a = PageAllocator(3)
    assert [a.allocate(), a.allocate(), a.allocate()] == [0, 1, 2] and a.num_free == 0
    with pytest.raises(OutOfPages):
        a.allocate()
    a.free(1)
    assert a.num_free == 1 and a.allocate() == 1
    a.incref(2)
    a.free(2)
    assert a.num_free == 0 and a.ref_count(2) == 1
    a.free(2)
    assert a.num_free == 1
    with pytest.raises(RuntimeError, match="double free"):
        a.free(2)
    with pytest.raises(RuntimeError, match="incref"):
        a.incref(2)
    with pytest.raises(RuntimeError, match="not in the pool"):
        a.free(7)


def test_tables_grow_one_page_per_boundary():
    # tests/cpp/test_paged_attention.cpp:47-81 and test_block_manager.cpp:10-60
    m = CacheManager([PagedNeed(2, 16)], page_size=4, num_pages=8, max_requests=2)
    a, b = m.open("a"), m.open("b")
    m.reserve(a, 5)
    m.commit(a, 5)
    assert a.tables[0] == [0, 1] and a.length == 5
    m.reserve(b, 4)
    m.commit(b, 4)
    assert b.tables[0] == [2] and not set(a.tables[0]) & set(b.tables[0])
    for _ in range(3):  # 6, 7, 8: still two pages
        m.reserve(a, 1)
        m.commit(a, 1)
    assert len(a.tables[0]) == 2
    m.reserve(a, 1)
    assert a.tables[0] == [0, 1, 3]
    assert m.pages_for(9) == 3 and m.free_pages() == 4
    assert m.can_reserve([(a, 4 * 3), (b, 4)]) and not m.can_reserve([(a, 4 * 3 + 1), (b, 5)])
    m.close(a)
    assert m.free_pages() == 7 and a.closed and a.tables[0] == []
    c = m.open("c")
    m.reserve(c, 1)
    assert c.tables[0] == [3]  # the page freed last is the next one handed out
    with pytest.raises(NoFreeSlot):
        m.open("d")
    with pytest.raises(RuntimeError, match="already open"):
        m.open("b")
    with pytest.raises(RuntimeError, match="closed twice"):
        m.close(a)
    m.check_invariants()


def test_reserve_fails_without_side_effects():
    m = CacheManager([PagedNeed(1, 8), PagedNeed(1, 8, window=4)], page_size=2, num_pages=[6, 2], max_requests=2)
    a = m.open("a")
    before = [list(t) for t in a.tables]
    with pytest.raises(OutOfPages, match="group 1"):
        m.reserve(a, 6)  # group 0 could hold it, group 1 cannot: nothing may be taken
    assert [list(t) for t in a.tables] == before and m.free_pages(0) == 6 and m.free_pages(1) == 2
    with pytest.raises(RuntimeError, match="beyond"):
        m.commit(a, 1)
    m.check_invariants()


def test_window_gives_pages_back():
    ps, w = 4, 6
    m = CacheManager([PagedNeed(1, 8), PagedNeed(1, 8, window=w)], page_size=ps, num_pages=[16, 5], max_requests=1)
    a = m.open("a")
    held_max = 0
    for step in range(40):
        n = [3, 1, 2, 5, 1][step % 5]
        if a.length + n > 64:
            break
        m.reserve(a, n)
        # every position the next queries read lies on a live page
        for p in range(a.length, a.length + n):
            for j in range(max(0, p - w + 1), p + 1):
                assert a.tables[1][j // ps] >= 0
        m.commit(a, n)
        dead = max(0, a.length - w + 1) // ps
        assert all(x == -1 for x in a.tables[1][:dead]) and all(x >= 0 for x in a.tables[1][dead:])
        assert all(x >= 0 for x in a.tables[0])
        held_max = max(held_max, a.pages_held(1))
        m.check_invariants()
    assert a.length > 40 and held_max <= 4  # the windowed group never needs the whole pool
    assert m.max_pages_held(1000, 5)[1] <= 5 and m.max_pages_held(1000, 5)[0] == 250
    m.close(a)
    assert m.free_pages(0) == 16 and m.free_pages(1) == 5


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_every_page_accounted(seed):
    rng = random.Random(seed)
    windowed = seed % 2 == 1
    groups = [PagedNeed(2, 16)] + ([PagedNeed(1, 32, window=5)] if windowed else [])
    m = CacheManager(groups, page_size=rng.choice([1, 3, 4, 8]), num_pages=rng.randint(6, 20), max_requests=4)
    live, next_id, events = {}, 0, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.free_slots:
            live[next_id] = m.open(next_id)
            next_id += 1
        elif op < 0.85 and live:
            rc = live[rng.choice(list(live))]
            n = rng.randint(1, 9)
            if m.can_reserve([(rc, n)]):
                m.reserve(rc, n)
                m.commit(rc, n)
                events += 1
            else:
                snapshot = ([list(t) for t in rc.tables], rc.length, [a.num_free for a in m.allocators])
                with pytest.raises(OutOfPages):
                    m.reserve(rc, n)
                assert snapshot == ([list(t) for t in rc.tables], rc.length, [a.num_free for a in m.allocators])
        elif live:
            m.close(live.pop(rng.choice(list(live))))
        m.check_invariants()
        for rc in live.values():
            assert len(rc.tables[0]) == m.pages_for(rc.length) or len(rc.tables[0]) >= m.pages_for(rc.length)
    for rc in list(live.values()):
        m.close(rc)
    m.check_invariants()
    assert all(a.num_free == a.num_pages for a in m.allocators) and m.free_slots == 4 and events > 50


def test_groups_with_page_geometries_of_their_own():
    """A need may say how many positions one of its entries holds and how many entries a page of
    its group has; the manager then counts that group's pages, and hands back a window's pages, by
    those numbers, beside a group that uses the cache's page size."""
    from dataclasses import dataclass
    from from_scratch_inference_engine_amd.cache.needs import CacheNeed

    @dataclass(frozen=True)
    class Blocks(CacheNeed):
        tokens_per_entry: int = 4
        page_entries: int = 2
        window: object = None

    m = CacheManager([PagedNeed(2, 8), Blocks(), Blocks(window=10)], page_size=4, num_pages=[16, 5, 5], max_requests=2)
    assert [m.tokens_per_page(g) for g in range(3)] == [4, 8, 8] and m.smallest_page_tokens == 4
    assert [m.pages_for(17, g) for g in range(3)] == [5, 3, 3]
    rc = m.open("r")
    assert m.new_pages_needed(rc, 17) == [5, 3, 3]
    assert m.max_pages_held(100, 6) == [25, 13, 4]      # the windowed group: 10 + 6 + 8 positions and one page
    m.reserve(rc, 17)
    m.commit(rc, 17)
    assert [len(t) for t in rc.tables] == [5, 3, 3]
    assert rc.tables[2][0] == -1 and rc.tables[2][1] >= 0  # positions before 17 - 10 + 1 = 8 are past the window: page 0 is back
    assert m.new_pages_needed(rc, 7) == [1, 0, 0] and m.new_pages_needed(rc, 8) == [2, 1, 1]
    with pytest.raises(RuntimeError, match="beyond the reserved"):
        m.commit(rc, 8)                                   # 25 positions do not fit five pages of four
    assert not m.can_reserve([(rc, 17 * 8)])
    m.check_invariants()
    m.close(rc)
    assert [a.num_free for a in m.allocators] == [16, 5, 5]


def test_pages_that_fit_the_free_memory():
    from from_scratch_inference_engine_amd.cache.manager import pages_that_fit

    gib = 1 << 30
    # nine tenths of 100 GiB less the reserve of 2 GiB, in pages of 16 tokens of 57,344 bytes
    assert pages_that_fit(100 * gib, 57344, 16) == (int(100 * gib * 0.9) - 2 * gib) // (57344 * 16)
    assert pages_that_fit(100 * gib, 57344, 16, fraction=0.5, reserve_bytes=0) == 50 * gib // (57344 * 16)
    assert pages_that_fit(gib, 57344, 16) == 1  # nothing left beside the reserve: one page, and the pool will say so
    with pytest.raises(ValueError):
        pages_that_fit(gib, 0, 16)
