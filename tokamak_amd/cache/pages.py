"""Page accounting: pools, cache groups, per-request block tables.

Positions map to pages as in the reference (src/tokamak/memory/block_manager.py:7):
position ``p`` lives in page ``table[p // page_size]`` at offset ``p % page_size``.
A *cache group* is a set of cache slots (layer calls) with the same retention
rule; each group has a pool and block tables of its own, so a group that only
needs a window of recent tokens gives pages back while a request is still
running (the mechanism of src/tokamak/memory/block_manager.py:95-129) without
touching the group that keeps everything.
"""

from __future__ import annotations

from dataclasses import dataclass

RELEASED = -1  # table entry of a page that was handed back behind a window


class OutOfPagesError(RuntimeError):
    """The pool cannot satisfy an allocation
    (reference: src/tokamak/memory/block_manager.py:21-26)."""


@dataclass(frozen=True)
class CacheGroupSpec:
    """``slots``: cache slots stored in this group's pages.  ``window``: None
    keeps every token; W keeps only what a query may still see when each query
    sees the last W positions (itself included)."""

    name: str
    slots: tuple[int, ...]
    window: int | None = None


class PagePool:
    """LIFO free list over ``num_pages`` page ids: freed pages are used again
    first (reference: src/tokamak/memory/block_manager.py:47-48,92-93)."""

    def __init__(self, num_pages: int) -> None:
        if num_pages < 1:
            raise ValueError(f"num_pages must be >= 1, got {num_pages}")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, count: int) -> list[int]:
        """``count`` pages, all or nothing."""
        if count > len(self._free):
            raise OutOfPagesError(
                f"need {count} page(s), but only {len(self._free)} of {self.num_pages} are free"
            )
        out = []
        for _ in range(count):
            page = self._free.pop()
            if self._held[page]:
                raise AssertionError(f"page {page} handed out twice")
            self._held[page] = True
            out.append(page)
        return out

    def give_back(self, pages) -> None:
        for page in pages:
            if not self._held[page]:
                raise AssertionError(f"page {page} freed twice")
            self._held[page] = False
            self._free.append(page)

    def check(self) -> None:
        """Every page is either free once or held once."""
        free = sorted(self._free)
        if len(set(free)) != len(free):
            raise AssertionError("a page is in the free list twice")
        for page in range(self.num_pages):
            if self._held[page] == (page in set(free)):
                raise AssertionError(f"page {page} is both held and free, or neither")


class GroupTables:
    """Block tables of one cache group."""

    def __init__(self, spec: CacheGroupSpec, num_pages: int, page_size: int) -> None:
        if page_size < 1:
            raise ValueError(f"page_size must be >= 1, got {page_size}")
        self.spec = spec
        self.page_size = page_size
        self.pool = PagePool(num_pages)
        self.tables: dict[object, list[int]] = {}
        self.first_live: dict[object, int] = {}  # logical pages below this were released

    def pages_needed(self, num_tokens: int) -> int:
        if num_tokens < 0:
            raise ValueError(f"num_tokens must be >= 0, got {num_tokens}")
        return -(-num_tokens // self.page_size)

    def shortfall(self, request, num_tokens: int) -> int:
        return max(0, self.pages_needed(num_tokens) - len(self.tables.get(request, ())))

    def grow(self, request, num_tokens: int) -> None:
        table = self.tables.setdefault(request, [])
        table.extend(self.pool.take(self.shortfall(request, num_tokens)))

    def release_before(self, request, first_needed_position: int) -> int:
        """Give back pages that lie wholly before ``first_needed_position``;
        their table entries become ``RELEASED``.  Monotonic and idempotent."""
        table = self.tables.get(request)
        if table is None:
            return 0
        lo = self.first_live.get(request, 0)
        hi = min(max(first_needed_position // self.page_size, lo), len(table))
        self.pool.give_back(table[i] for i in range(lo, hi))
        for i in range(lo, hi):
            table[i] = RELEASED
        if hi > lo:
            self.first_live[request] = hi
        return hi - lo

    def releasable_before(self, request, first_needed_position: int) -> int:
        """How many pages ``release_before`` would give back now."""
        table = self.tables.get(request)
        if table is None:
            return 0
        lo = self.first_live.get(request, 0)
        return min(max(first_needed_position // self.page_size, lo), len(table)) - lo

    def free(self, request) -> None:
        table = self.tables.pop(request, None)
        self.first_live.pop(request, None)
        if table:
            self.pool.give_back(p for p in table if p != RELEASED)

    def live_pages(self, request) -> int:
        return sum(1 for p in self.tables.get(request, ()) if p != RELEASED)
