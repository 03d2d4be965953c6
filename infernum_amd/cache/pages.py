"""Bookkeeping of pages on the host: which are free, which a request holds.

A LIFO stack of free page numbers, ``allocate`` returning nothing when it is
empty, and a loud failure on a double free or a page outside the pool, as
infernum/src/block_allocator.rs:27-110; the in-use flags make the double-free
check O(1).  A request's pages per group are a block table: page numbers in the
order of positions, ``page_size`` tokens each (block_allocator.rs:119-198).
"""
from __future__ import annotations

from typing import List, Optional

NO_PAGE = -1


class PageError(RuntimeError):
    """A page was freed twice, was never part of the pool, or is not held."""


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = int(num_pages)
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))   # pop() gives 0 first
        self._in_use = bytearray(self.num_pages)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def can_allocate(self, n: int) -> bool:
        return n <= len(self._free)

    def allocate(self) -> Optional[int]:
        if not self._free:
            return None
        p = self._free.pop()
        self._in_use[p] = 1
        return p

    def allocate_many(self, n: int) -> Optional[List[int]]:
        """n pages or none at all."""
        if n > len(self._free):
            return None
        return [self.allocate() for _ in range(n)]

    def free(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise PageError(f"page {page} is outside the pool of {self.num_pages}")
        if not self._in_use[page]:
            raise PageError(f"page {page} is freed twice")
        self._in_use[page] = 0
        self._free.append(page)

    def is_used(self, page: int) -> bool:
        return bool(self._in_use[page])


def pages_for(num_tokens: int, page_size: int) -> int:
    return (num_tokens + page_size - 1) // page_size


class BlockTable:
    """Pages of one request in one group.  ``pages[i]`` holds positions
    [i * page_size, (i + 1) * page_size); NO_PAGE where a window has passed."""

    __slots__ = ("pages", "num_tokens", "first_live")

    def __init__(self) -> None:
        self.pages: List[int] = []
        self.num_tokens = 0
        self.first_live = 0      # pages before this index have been given back

    def live_pages(self) -> List[int]:
        return [p for p in self.pages[self.first_live:] if p != NO_PAGE]
