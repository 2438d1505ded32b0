"""Page allocator with reference counts.

The reference's allocator is a LIFO stack of one-token slots, all-or-nothing ``alloc(n)`` and a
``free`` that trusts its caller (ullm/core/kv_cache.py:118-134).  Here the unit is a page of
``page_size`` tokens and every page carries a count of its holders (block tables of requests and
the prefix tree), so a shared page survives until its last holder lets go and a double free is an
error instead of a silent corruption.
"""
from __future__ import annotations

from typing import List, Optional


class PageError(RuntimeError):
    """Bookkeeping was violated (double free, unknown page)."""


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() hands out page 0 first
        self._ref: List[int] = [0] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> Optional[List[int]]:
        """``n`` pages with one holder each, or None if fewer than ``n`` are free (nothing taken)."""
        if n < 0:
            raise ValueError("negative page count")
        if n > len(self._free):
            return None
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._ref[p] = 1
        return pages

    def incref(self, page: int) -> None:
        if not (0 <= page < self.num_pages) or self._ref[page] <= 0:
            raise PageError(f"incref of page {page} that nobody holds")
        self._ref[page] += 1

    def decref(self, page: int) -> bool:
        """Drop one holder; returns True if the page went back to the free list."""
        if not (0 <= page < self.num_pages) or self._ref[page] <= 0:
            raise PageError(f"page {page} freed more often than it was held")
        self._ref[page] -= 1
        if self._ref[page] == 0:
            self._free.append(page)
            return True
        return False

    def refcount(self, page: int) -> int:
        return self._ref[page]

    def check(self) -> None:
        held = sum(1 for r in self._ref if r > 0)
        if held + len(self._free) != self.num_pages:
            raise PageError(f"{held} held + {len(self._free)} free != {self.num_pages} pages")
        if len(set(self._free)) != len(self._free):
            raise PageError("a page is on the free list twice")
        for p in self._free:
            if self._ref[p] != 0:
                raise PageError(f"free page {p} has {self._ref[p]} holders")
