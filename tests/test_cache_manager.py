"""The cache manager on the CPU: no page lost, held twice or freed twice, under random orders."""
from __future__ import annotations

import random

import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from tokenmill_amd.cache import (RELEASED, AllocStatus, CacheManager, OutOfPages, PageAllocator, SlotAllocator)


def test_allocator_basics_and_fifo_reuse():
    """reference tests/test_block_allocator.py:13-22 and src/infer/kv/block_allocator.py:39-64"""
    a = PageAllocator(4)
    assert a.allocate(3) == [0, 1, 2] and a.num_free == 1
    with pytest.raises(OutOfPages):
        a.allocate(2)
    assert a.num_free == 1                                  # nothing was taken by the failed call
    a.release([1])
    with pytest.raises(RuntimeError, match="double free"):
        a.release([1])
    assert a.allocate(2) == [3, 1]                          # a returned page comes back after the list wraps
    a.check_invariants()
    a.share(3)
    a.release([3])
    assert a.refcount[3] == 1 and 3 not in a.free
    a.release([3, 0, 2, 1])
    assert a.num_free == 4
    a.check_invariants()


def test_state_slots():
    s = SlotAllocator(2)
    x, y = s.allocate(), s.allocate()
    assert {x, y} == {0, 1}
    with pytest.raises(OutOfPages):
        s.allocate()
    s.release(x)
    with pytest.raises(RuntimeError, match="double free"):
        s.release(x)
    assert s.allocate() == x
    s.check_invariants()


def test_page_arithmetic_and_growth():
    """reference tests/test_scheduler.py:42-52,110-120: 5 tokens at page size 4 hold 2 pages; the
    second page appears exactly when the length reaches 5."""
    m = CacheManager([None], num_pages=16, page_size=4, num_state_slots=4)
    rc = m.allocate("a", 4)
    assert len(rc.tables[0]) == 1
    assert m.can_append(rc, 5)
    m.append(rc, 5)
    assert len(rc.tables[0]) == 2
    m.append(rc, 6)
    assert len(rc.tables[0]) == 2
    t = rc.tables[0]
    assert m.slot(rc, 0, 5) == t[1] * 4 + 1 and m.slot(rc, 0, 3) == t[0] * 4 + 3
    m.free(rc)
    with pytest.raises(RuntimeError, match="double free"):
        m.free(rc)
    assert m.num_free_pages == 16
    m.check_invariants()


def test_admission_respects_the_watermark():
    """reference tests/test_scheduler.py:55-66: 10 pages, watermark 0.2 admits 7 + 1 but not 7 + 2."""
    m = CacheManager([None], 10, 4, 8, watermark=0.2)
    assert m.allocation_status(28) == AllocStatus.OK
    m.allocate("a", 28)
    assert m.allocation_status(4) == AllocStatus.OK           # 3 - 1 = 2 >= 2
    assert m.allocation_status(8) == AllocStatus.LATER        # 3 - 2 = 1 < 2
    assert m.allocation_status(4 * 9) == AllocStatus.NEVER    # 9 + 2 > 10
    m2 = CacheManager([None], 4, 4, 8)
    assert m2.allocation_status(4 * 5) == AllocStatus.NEVER   # reference tests/test_scheduler.py:102-107


def test_groups_have_pages_of_their_own_and_a_window_gives_pages_back():
    m = CacheManager([None, 8], num_pages=[8, 4], page_size=4, num_state_slots=2)
    rc = m.allocate("a", 14)                                   # 4 pages in each group
    assert [len(t) for t in rc.tables] == [4, 4]
    assert m.allocators[0].num_free == 4 and m.allocators[1].num_free == 0
    assert m.allocation_status(4) == AllocStatus.LATER         # the windowed group is full
    # 14 tokens cached; the next query (position 14) sees keys 7..14: page 0 (0..3) is behind, page 1 (4..7) is not
    assert m.release_behind_window(rc, 14) == 1
    assert rc.tables[1][0] == RELEASED and rc.tables[1][1] != RELEASED and rc.tables[0][0] != RELEASED
    assert m.release_behind_window(rc, 14) == 0                # nothing is given back twice
    with pytest.raises(RuntimeError, match="window has passed"):
        m.slot(rc, 1, 2)
    m.check_invariants()
    m.append(rc, 17)                                           # a fifth page; the windowed group reuses the freed one
    assert len(rc.tables[1]) == 5
    m.release_behind_window(rc, 17)                            # keys 10..: pages 0, 1 (4..7) gone
    assert rc.tables[1][:2] == [RELEASED, RELEASED]
    m.check_invariants()
    m.free(rc)
    assert m.allocators[0].num_free == 8 and m.allocators[1].num_free == 4
    m.check_invariants()


def test_all_groups_or_none():
    m = CacheManager([None, None], num_pages=[8, 2], page_size=4, num_state_slots=2)
    with pytest.raises(OutOfPages):
        m.allocate("a", 12)                                    # 3 pages: the second group has 2
    assert m.allocators[0].num_free == 8 and m.allocators[1].num_free == 2 and m.slots.num_free == 2
    rc = m.allocate("b", 8)
    assert not m.can_append(rc, 9)
    with pytest.raises(OutOfPages):
        m.append(rc, 9)
    assert [len(t) for t in rc.tables] == [2, 2]               # the first group did not grow alone
    m.check_invariants()


@settings(max_examples=200, deadline=None)
@given(st.lists(st.tuples(st.integers(0, 4), st.integers(0, 7), st.integers(1, 40)), max_size=80), st.integers(0, 3))
def test_random_orders_of_requests(ops, seed):
    """Random admissions, growth, window releases and frees: the invariants hold after every
    operation and every page is back at the end (reference tests/test_block_allocator.py:25-47)."""
    rng = random.Random(seed)
    m = CacheManager([None, 12], num_pages=[24, 24], page_size=4, num_state_slots=5, watermark=0.05)
    length: dict[str, int] = {}
    for kind, who, n in ops:
        rid = f"r{who}"
        if kind in (0, 1):
            if rid not in m.live:
                if m.allocation_status(n) == AllocStatus.OK:
                    m.allocate(rid, n)
                    length[rid] = n
                elif any(m.pages_for(n) > a.num_free for a in m.allocators) or m.slots.num_free < 1:
                    with pytest.raises(OutOfPages):        # (otherwise only the watermark holds it back)
                        m.allocate(rid, n)
        elif kind == 2 and rid in m.live:
            rc = m.live[rid]
            new = length[rid] + rng.randint(1, 9)
            if m.can_append(rc, new):
                m.append(rc, new)
                length[rid] = new
            else:
                with pytest.raises(OutOfPages):
                    m.append(rc, new)
        elif kind == 3 and rid in m.live:
            m.release_behind_window(m.live[rid], length[rid])
        elif kind == 4 and rid in m.live:
            m.free(m.live[rid])
            del length[rid]
        m.check_invariants()
        for r, rc in m.live.items():
            assert len(rc.tables[0]) >= m.pages_for(length[r])
    for rc in list(m.live.values()):
        m.free(rc)
    m.check_invariants()
    assert [a.num_free for a in m.allocators] == [24, 24] and m.slots.num_free == 5
