"""The cache manager: who holds which pages and which state slot. It never touches the GPU.

Layer groups. Cache layers with the same needs (kv heads, head size, and whether they keep every
token or a window of the last W) form a group; each group has a page pool of its own and every
live request has one block table per group. The reference has a single group that keeps
everything (reference src/infer/kv/paged_cache.py:55-137); its rules are kept for each group:

  position p of a request lives in flat slot  table[p // page] * page + p % page     (:90-91)
  admission: need = ceil(tokens / page) per group; NEVER if need + watermark pages > pool,
             OK if free - need >= watermark pages, else LATER; all groups or none       (:95-102)
  admission takes pages for all tokens at once                                            (:104-123)
  growth: one more page when the length crosses a page edge; growth ignores the watermark (:125-131)
  the end of a request gives every page back, last page first                             (:133-137)

Beyond the reference: a windowed group also gives a page back as soon as the window has passed
it (``release_behind_window``), and every request holds one state slot for per-request state of
fixed size, taken with its first pages and returned with them.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, field

from tokenmill_amd.cache.allocator import OutOfPages, PageAllocator, SlotAllocator

RELEASED = -1       # a block-table entry whose page the window has passed


class AllocStatus(enum.Enum):
    OK = 0
    LATER = 1       # not enough free pages now
    NEVER = 2       # would not fit even in an empty pool


@dataclass
class RequestCache:
    """What one live request holds."""
    request_id: str
    tables: list[list[int]]                     # per group: page ids by logical page index
    state_slot: int
    released: list[int] = field(default_factory=list)   # per group: leading pages already given back
    fresh: bool = True                          # state slot not yet zeroed for this admission

    def capacity(self, page_size: int) -> int:
        return min(len(t) for t in self.tables) * page_size if self.tables else 1 << 60


class CacheManager:
    def __init__(self, group_windows: list[int | None], num_pages: int | list[int], page_size: int,
                 num_state_slots: int, watermark: float = 0.0):
        if page_size < 1:
            raise ValueError("page_size must be at least 1")
        self.page_size = page_size
        self.windows = list(group_windows)
        self.any_window = any(w is not None for w in self.windows)
        counts = [num_pages] * len(self.windows) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(self.windows):
            raise ValueError("one page count per group")
        self.allocators = [PageAllocator(n) for n in counts]
        self.watermark_pages = [int(watermark * n) for n in counts]
        self.slots = SlotAllocator(num_state_slots)
        self.live: dict[str, RequestCache] = {}

    # --- facts --------------------------------------------------------------------------------------

    @property
    def num_groups(self) -> int:
        return len(self.allocators)

    def pages_for(self, num_tokens: int) -> int:
        return -(-num_tokens // self.page_size)

    @property
    def num_free_pages(self) -> int:
        """Free pages of the tightest group (all groups are equal when there is one)."""
        return min((a.num_free for a in self.allocators), default=0)

    @property
    def num_pages(self) -> int:
        return min((a.num_pages for a in self.allocators), default=0)

    def usage(self) -> float:
        return max((a.num_used / a.num_pages for a in self.allocators), default=0.0)

    def slot(self, rc: RequestCache, group: int, pos: int) -> int:
        page = rc.tables[group][pos // self.page_size]
        if page == RELEASED:
            raise RuntimeError(f"{rc.request_id}: position {pos} lies in a page the window has passed")
        return page * self.page_size + pos % self.page_size

    # --- admission, growth, release -------------------------------------------------------------------

    def allocation_status(self, num_tokens: int) -> AllocStatus:
        need = self.pages_for(num_tokens)
        if any(need + wm > a.num_pages for a, wm in zip(self.allocators, self.watermark_pages)):
            return AllocStatus.NEVER
        if self.slots.num_free < 1:
            return AllocStatus.LATER
        if all(a.num_free - need >= wm for a, wm in zip(self.allocators, self.watermark_pages)):
            return AllocStatus.OK
        return AllocStatus.LATER

    def allocate(self, request_id: str, num_tokens: int) -> RequestCache:
        """Pages for ``num_tokens`` tokens in every group and a state slot; all or nothing."""
        if request_id in self.live:
            raise RuntimeError(f"{request_id} still holds pages")
        need = self.pages_for(num_tokens)
        if any(need > a.num_free for a in self.allocators) or self.slots.num_free < 1:
            raise OutOfPages(f"{request_id}: need {need} pages per group and a state slot")
        rc = RequestCache(request_id, [a.allocate(need) for a in self.allocators], self.slots.allocate(),
                          [0] * self.num_groups)
        self.live[request_id] = rc
        return rc

    def can_append(self, rc: RequestCache, length: int) -> bool:
        """Room for ``length`` tokens, with at most the pages that are free now?"""
        need = self.pages_for(length)
        return all(len(t) >= need or a.num_free >= need - len(t) for t, a in zip(rc.tables, self.allocators))

    def append(self, rc: RequestCache, length: int) -> None:
        """Grow every table to hold ``length`` tokens; all or nothing."""
        if not self.try_append(rc, length):
            raise OutOfPages(f"{rc.request_id}: cannot grow to {length} tokens")

    def try_append(self, rc: RequestCache, length: int) -> bool:
        """``append`` if there is room, all or nothing; False (nothing changed) if there is not."""
        need = -(-length // self.page_size)
        tables, allocators = rc.tables, self.allocators
        short = False
        for t, a in zip(tables, allocators):
            if len(t) < need:
                if a.num_free < need - len(t):
                    return False
                short = True
        if short:
            for t, a in zip(tables, allocators):
                if len(t) < need:
                    t.extend(a.allocate(need - len(t)))
        return True

    def release_behind_window(self, rc: RequestCache, num_computed: int) -> int:
        """Give back, in windowed groups, the pages that no later token can see: with
        ``num_computed`` tokens cached, the next query sits at position >= num_computed and sees
        keys from num_computed - W + 1 on. Returns the number of pages given back."""
        given = 0
        if not self.any_window:
            return given
        for g, window in enumerate(self.windows):
            if window is None:
                continue
            first_needed = max(0, num_computed - window + 1)
            upto = min(first_needed // self.page_size, len(rc.tables[g]))
            table = rc.tables[g]
            back = [table[i] for i in range(rc.released[g], upto) if table[i] != RELEASED]
            for i in range(rc.released[g], upto):
                table[i] = RELEASED
            if upto > rc.released[g]:
                rc.released[g] = upto
            self.allocators[g].release(back)
            given += len(back)
        return given

    def free(self, rc: RequestCache) -> None:
        if self.live.get(rc.request_id) is not rc:
            raise RuntimeError(f"double free of request {rc.request_id}")
        for t, a in zip(rc.tables, self.allocators):
            a.release([p for p in reversed(t) if p != RELEASED])
            t.clear()
        self.slots.release(rc.state_slot)
        rc.state_slot = -1
        del self.live[rc.request_id]

    # --- checks -----------------------------------------------------------------------------------------

    def check_invariants(self) -> None:
        for g, a in enumerate(self.allocators):
            a.check_invariants()
            held: dict[int, int] = {}
            for rc in self.live.values():
                for p in rc.tables[g]:
                    if p != RELEASED:
                        held[p] = held.get(p, 0) + 1
            for p in range(a.num_pages):
                assert a.refcount[p] == held.get(p, 0), \
                    f"group {g} page {p}: refcount {a.refcount[p]} but held {held.get(p, 0)} times"
        self.slots.check_invariants()
        slots = [rc.state_slot for rc in self.live.values()]
        assert len(set(slots)) == len(slots), "a state slot is held by two requests"
        assert self.slots.num_slots - self.slots.num_free == len(slots), "a state slot was lost"
