"""Host-side bookkeeping of the cache: slots for sequences and pages for their keys/values.

Reference: the reference keeps one sequence, as one block per layer of ``max_seq_len``
rows taken from a pool with a free list (``src/kvcache/manager.zig:100-185``,
``src/kvcache/block_allocator.zig:30-102``, ``src/models/gemma3.zig:234-245``).  Here a
sequence holds a *slot* while it lives, and each *group* of layers with the same needs has
a pool of pages of 64 positions of its own.  A group that needs all keys keeps every page
of a sequence; a group whose layers look back at most ``window`` positions gives pages
back as soon as no later query can reach them, so such a sequence never holds more than
``window/64 + 2`` pages of that group.

Nothing here touches the GPU: the classes only decide which page holds which positions.
The device sees the outcome as a table per step (:meth:`GroupPages.plan`).
"""
from __future__ import annotations

import heapq
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

PAGE = 64   # positions per page


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


class OutOfSlots(CacheError):
    pass


class PagePool:
    """Free list over ``n_pages`` page ids.  Freed pages
    are handed out again, lowest id first, so a finished batch's pages are used again."""

    def __init__(self, n_pages: int):
        if n_pages < 1:
            raise CacheError(f"a page pool needs at least one page, got {n_pages}")
        self.n_pages = n_pages
        self._free: List[int] = list(range(n_pages))      # a heap: lowest id first
        self._held = [False] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages(f"all {self.n_pages} cache pages are in use")
        p = heapq.heappop(self._free)
        self._held[p] = True
        return p

    def free(self, page: int) -> None:
        if not (0 <= page < self.n_pages) or not self._held[page]:
            raise CacheError(f"page {page} freed although it is not held")
        self._held[page] = False
        heapq.heappush(self._free, page)


class SlotTable:
    """Slots for live sequences; each has its length."""

    def __init__(self, max_slots: int):
        if max_slots < 1:
            raise CacheError(f"need at least one slot, got {max_slots}")
        self.max_slots = max_slots
        self._free: List[int] = list(range(max_slots))    # a heap: lowest id first
        self.length: List[Optional[int]] = [None] * max_slots     # None: slot is free

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfSlots(f"all {self.max_slots} sequence slots are in use")
        s = heapq.heappop(self._free)
        self.length[s] = 0
        return s

    def free(self, slot: int) -> None:
        self.check(slot)
        self.length[slot] = None
        heapq.heappush(self._free, slot)

    def check(self, slot: int) -> None:
        if not (0 <= slot < self.max_slots) or self.length[slot] is None:
            raise CacheError(f"slot {slot} is not held")


@dataclass(frozen=True)
class GroupKey:
    """What a layer's cache needs; layers with equal keys share a group."""
    window: Optional[int]      # None: all keys
    n_kv_heads: int
    head_dim: int


def pages_in_reach(window: Optional[int], max_context: int, max_new: int = 1) -> int:
    """Most pages one sequence holds in a group while a step brings it up to ``max_new`` tokens,
    for sequences of at most ``max_context`` positions.  A group that needs all keys holds the
    whole context.  A window of W reaches back W - 1 positions from the step's first token, so
    the step spans W + max_new - 1 positions, which touch at most one page more than they fill."""
    full = (max_context + PAGE - 1) // PAGE
    if window is None:
        return full
    return min(full, (window + max_new - 1 + PAGE - 2) // PAGE + 1)


def pool_pages(window: Optional[int], max_slots: int, max_context: int, piece: int) -> int:
    """Pages a group's pool needs so that ``max_slots`` sequences of up to ``max_context``
    positions always fit when no step brings a sequence more than ``piece`` tokens: all keys of
    every sequence for a group without a window, only the window's reach plus the step's own
    tokens for a windowed one (what the reference's ring of W rows per sliding layer bounds)."""
    return max_slots * pages_in_reach(window, max_context, max(1, min(piece, max_context)))


class GroupPages:
    """The pages of one group: for every slot a map from page index (position // 64) to
    page id."""

    def __init__(self, key: GroupKey, n_pages: int, max_slots: int):
        self.key = key
        self.pool = PagePool(n_pages)
        self._pages: List[Dict[int, int]] = [dict() for _ in range(max_slots)]

    # the lowest page index that a query at position >= ``length`` can still reach
    def _first_needed(self, length: int) -> int:
        if self.key.window is None:
            return 0
        return max(0, length - self.key.window + 1) // PAGE

    def table_width(self, max_context: int, max_new: int = 1) -> int:
        """Columns that a step's table needs at most for sequences up to ``max_context``
        positions when a step brings up to ``max_new`` tokens per sequence."""
        return pages_in_reach(self.key.window, max_context, max_new)

    def plan(self, slot: int, pos0: int, n_new: int) -> Tuple[int, List[int]]:
        """Make sure pages exist for positions ``pos0 .. pos0+n_new-1`` and return
        ``(base, pages)``: ``pages[i]`` is the page id of page index ``base + i``, from the
        oldest page a query of this step can reach to the newest page it writes."""
        if n_new < 1:
            raise CacheError("a step brings at least one token per sequence")
        held = self._pages[slot]
        first_new, last_new = pos0 // PAGE, (pos0 + n_new - 1) // PAGE
        fresh = [i for i in range(first_new, last_new + 1) if i not in held]
        if len(fresh) > self.pool.n_free:
            raise OutOfPages(f"step needs {len(fresh)} more cache pages, {self.pool.n_free} are free "
                             f"of {self.pool.n_pages}")
        for i in fresh:
            held[i] = self.pool.alloc()
        base = self._first_needed(pos0)
        missing = [i for i in range(base, last_new + 1) if i not in held]
        if missing:
            raise CacheError(f"slot {slot}: pages {missing} within reach are not held")
        return base, [held[i] for i in range(base, last_new + 1)]

    def commit(self, slot: int, new_length: int) -> None:
        """After a step: give back the pages that no later query reaches."""
        held = self._pages[slot]
        keep_from = self._first_needed(new_length)
        for i in [i for i in held if i < keep_from]:
            self.pool.free(held.pop(i))

    def release(self, slot: int) -> None:
        held = self._pages[slot]
        for i in list(held):
            self.pool.free(held.pop(i))

    def held(self, slot: int) -> Dict[int, int]:
        return dict(self._pages[slot])
