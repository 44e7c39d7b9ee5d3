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
    # A query sees only the keys of its own chunk of this many positions (chunks are counted from
    # position 0 of the sequence); None: no chunks.  Pages of chunks that are over are given back.
    chunk: Optional[int] = None
    v_head_dim: Optional[int] = None   # size of a value head if it differs from the keys'
    # "tiles": K [page, kv head, 64, head_dim] and V transposed [page, kv head, head_dim, 64], in the
    # matrix cores' operand order where the sizes allow; "rows": K and V row by row,
    # [page, kv head, 64, head_dim] and [page, kv head, 64, v_head_dim], never reordered; "rows_vt": K row by
    # row and V transposed inside a page, [page, kv head, v_head_dim, 64] (a value column's 64 positions in a row)
    layout: str = "tiles"
    # The first positions of a sequence that stay visible whatever the window: the pages that hold them
    # are never given back, and stand in the first columns of a step's table row (``kept_pages``).
    keep_first: int = 0

    @property
    def kept_pages(self) -> int:
        """Pages at a sequence's start that are held for good (0 without a window: every page is)."""
        return (self.keep_first + PAGE - 1) // PAGE if (self.keep_first > 0 and self.reach is not None) else 0

    def covering(self, other: "GroupKey") -> Optional["GroupKey"]:
        """The need that serves this one and ``other`` on the same pages (two mixers that read one memory with
        different windows): the wider window, the larger count of kept positions.  None if sizes, chunk or
        layout differ."""
        same = (self.n_kv_heads, self.head_dim, self.chunk, self.v_head_dim, self.layout) == \
               (other.n_kv_heads, other.head_dim, other.chunk, other.v_head_dim, other.layout)
        if not same:
            return None
        window = None if (self.window is None or other.window is None) else max(self.window, other.window)
        return GroupKey(window, self.n_kv_heads, self.head_dim, self.chunk, self.v_head_dim, self.layout,
                        max(self.keep_first, other.keep_first))

    @property
    def reach(self) -> Optional[int]:
        """Positions a query looks back over at most, itself included (None: all of them)."""
        bounds = [b for b in (self.window, self.chunk) if b is not None]
        return min(bounds) if bounds else None

    def first_needed(self, length: int) -> int:
        """The oldest position that a query at position >= ``length`` can still see."""
        lo = 0
        if self.window is not None:
            lo = max(lo, length - self.window + 1)
        if self.chunk is not None:
            lo = max(lo, (length // self.chunk) * self.chunk)
        return lo


def pages_in_reach(window: Optional[int], max_context: int, max_new: int = 1, kept_pages: int = 0) -> int:
    """Most pages one sequence holds in a group while a step brings it up to ``max_new`` tokens,
    for sequences of at most ``max_context`` positions.  A group that needs all keys holds the
    whole context.  A window of W reaches back W - 1 positions from the step's first token, so
    the step spans W + max_new - 1 positions, which touch at most one page more than they fill.
    ``kept_pages``: pages at the sequence's start that a windowed group holds besides."""
    full = (max_context + PAGE - 1) // PAGE
    if window is None:
        return full
    return min(full, (window + max_new - 1 + PAGE - 2) // PAGE + 1 + kept_pages)


def pool_pages(window: Optional[int], max_slots: int, max_context: int, piece: int, kept_pages: int = 0) -> int:
    """Pages a group's pool needs so that ``max_slots`` sequences of up to ``max_context``
    positions always fit when no step brings a sequence more than ``piece`` tokens: all keys of
    every sequence for a group without a window, only the window's reach plus the step's own
    tokens for a windowed one (what the reference's ring of W rows per sliding layer bounds)."""
    return max_slots * pages_in_reach(window, max_context, max(1, min(piece, max_context)), kept_pages)


class GroupPages:
    """The pages of one group: for every slot a map from page index (position // 64) to
    page id."""

    def __init__(self, key: GroupKey, n_pages: int, max_slots: int):
        self.key = key
        self.pool = PagePool(n_pages)
        self._pages: List[Dict[int, int]] = [dict() for _ in range(max_slots)]

    # the lowest page index that a query at position >= ``length`` can still reach
    def _first_needed(self, length: int) -> int:
        return self.key.first_needed(length) // PAGE

    def table_width(self, max_context: int, max_new: int = 1) -> int:
        """Columns that a step's table needs at most for sequences up to ``max_context``
        positions when a step brings up to ``max_new`` tokens per sequence."""
        return pages_in_reach(self.key.reach, max_context, max_new, self.key.kept_pages)

    def plan(self, slot: int, pos0: int, n_new: int) -> Tuple[int, List[int]]:
        """Make sure pages exist for positions ``pos0 .. pos0+n_new-1`` and return
        ``(base, pages)``: ``pages[i]`` is the page id of page index ``base + i``, from the
        oldest page a query of this step can reach to the newest page it writes.  In a group that
        keeps a sequence's first pages (``key.kept_pages`` = k > 0) those come first: ``pages[i]`` is
        page index i for i < k, and page index ``base + i - k`` from there on, with ``base >= k``."""
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
        kept = self.key.kept_pages
        base = max(self._first_needed(pos0), kept)
        wanted = list(range(0, min(kept, last_new + 1))) + list(range(base, last_new + 1))
        missing = [i for i in wanted if i not in held]
        if missing:
            raise CacheError(f"slot {slot}: pages {missing} within reach are not held")
        return base, [held[i] for i in wanted]

    def commit(self, slot: int, new_length: int) -> None:
        """After a step: give back the pages that no later query reaches."""
        held = self._pages[slot]
        keep_from = self._first_needed(new_length)
        kept = self.key.kept_pages
        for i in [i for i in held if kept <= i < keep_from]:
            self.pool.free(held.pop(i))

    def release(self, slot: int) -> None:
        held = self._pages[slot]
        for i in list(held):
            self.pool.free(held.pop(i))

    def held(self, slot: int) -> Dict[int, int]:
        return dict(self._pages[slot])
