"""Free list of cache pages with reference counts, and the pool of per-request state slots.

Same contract as the reference's BlockAllocator without its prefix-cache extras (reference
src/infer/kv/block_allocator.py:19-87): pages are handed out from the front of a FIFO free list and
returned to its back, so a returned page is used again once the list has wrapped; ``allocate``
takes nothing when it cannot take everything; releasing a free page is an error.
"""
from __future__ import annotations

from collections import deque


class OutOfPages(RuntimeError):
    pass


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self.free: deque[int] = deque(range(num_pages))
        self.refcount = [0] * num_pages

    @property
    def num_free(self) -> int:
        return len(self.free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self.free)

    def allocate(self, n: int) -> list[int]:
        if n > len(self.free):
            raise OutOfPages(f"need {n} pages, {len(self.free)} free")
        ids = []
        for _ in range(n):
            p = self.free.popleft()
            if self.refcount[p] != 0:
                raise RuntimeError(f"page {p} handed out twice")
            self.refcount[p] = 1
            ids.append(p)
        return ids

    def share(self, page: int) -> None:
        """One more holder of a page that is in use."""
        if self.refcount[page] <= 0:
            raise RuntimeError(f"page {page} is free and cannot be shared")
        self.refcount[page] += 1

    def release(self, ids) -> None:
        for p in ids:
            if not 0 <= p < self.num_pages or self.refcount[p] <= 0:
                raise RuntimeError(f"double free of page {p}")
            self.refcount[p] -= 1
            if self.refcount[p] == 0:
                self.free.append(p)

    def check_invariants(self) -> None:
        free = set(self.free)
        assert len(free) == len(self.free), "a page is in the free list twice"
        for p in range(self.num_pages):
            assert (self.refcount[p] == 0) == (p in free), f"page {p}: refcount {self.refcount[p]}, free {p in free}"
        assert len(free) + sum(1 for r in self.refcount if r > 0) == self.num_pages


class SlotAllocator:
    """One slot index per live request for state of fixed size (the idea of the reference's
    contiguous baseline: a slot taken at admission and returned at the end,
    reference src/infer/kv/contiguous.py:56-71)."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free: deque[int] = deque(range(num_slots))
        self.held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self.free)

    def allocate(self) -> int:
        if not self.free:
            raise OutOfPages("no state slot free")
        s = self.free.popleft()
        if self.held[s]:
            raise RuntimeError(f"state slot {s} handed out twice")
        self.held[s] = True
        return s

    def release(self, s: int) -> None:
        if not 0 <= s < self.num_slots or not self.held[s]:
            raise RuntimeError(f"double free of state slot {s}")
        self.held[s] = False
        self.free.append(s)

    def check_invariants(self) -> None:
        free = set(self.free)
        assert len(free) == len(self.free), "a state slot is in the free list twice"
        for s in range(self.num_slots):
            assert self.held[s] != (s in free), f"state slot {s}: held {self.held[s]}, free {s in free}"
