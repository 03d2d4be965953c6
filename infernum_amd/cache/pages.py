"""Bookkeeping of pages on the host: which are free, which a request holds.

A LIFO stack of free page numbers, ``allocate`` returning nothing when it is
empty, and a loud failure on a double free or a page outside the pool, as
infernum/src/block_allocator.rs:27-110; the in-use flags make the double-free
check O(1).  A request's pages per group are a block table: page numbers in the
order of positions, ``page_size`` tokens each (block_allocator.rs:119-198).

The bookkeeping itself is native (``csrc/host_core.cpp``); the classes here are
its Python face.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional

from . import native

NO_PAGE = -1


class PageError(RuntimeError):
    """A page was freed twice, was never part of the pool, or is not held."""


class PageAllocator:
    """A pool of ``num_pages`` pages; ``_view`` wraps a pool that a cache manager (``_owner``, kept alive by
    this object) owns."""

    def __init__(self, num_pages: int, _view: Optional[int] = None, _owner: object = None):
        self._lib = native.lib()
        self._owner = _owner
        if _view is not None:
            self._h, self._owned = ctypes.c_void_p(_view), False
        else:
            if num_pages <= 0:
                raise ValueError("a page pool needs at least one page")
            self._h, self._owned = ctypes.c_void_p(self._lib.ia_pool_create(int(num_pages))), True
        self.num_pages = int(self._lib.ia_pool_num_pages(self._h))

    def __del__(self):
        if getattr(self, "_owned", False) and self._h:
            self._lib.ia_pool_destroy(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return int(self._lib.ia_pool_num_free(self._h))

    @property
    def num_used(self) -> int:
        return self.num_pages - self.num_free

    def can_allocate(self, n: int) -> bool:
        return n <= self.num_free

    def allocate(self) -> Optional[int]:
        p = int(self._lib.ia_pool_allocate(self._h))
        return None if p < 0 else p

    def allocate_many(self, n: int) -> Optional[List[int]]:
        """n pages or none at all."""
        out = (ctypes.c_int * max(n, 1))()
        if not self._lib.ia_pool_allocate_many(self._h, int(n), out):
            return None
        return list(out[:n])

    def free(self, page: int) -> None:
        if self._lib.ia_pool_free(self._h, int(page)) != 0:
            raise PageError(self._lib.ia_pool_error(self._h).decode())

    def is_used(self, page: int) -> bool:
        return bool(self._lib.ia_pool_is_used(self._h, int(page)))


def pages_for(num_tokens: int, page_size: int) -> int:
    return (num_tokens + page_size - 1) // page_size


class BlockTable:
    """Pages of one request in one group (a copy of the native table at the time it was asked for).
    ``pages[i]`` holds positions [i * page_size, (i + 1) * page_size); NO_PAGE where a window has passed."""

    __slots__ = ("pages", "num_tokens", "first_live")

    def __init__(self, pages: Optional[List[int]] = None, num_tokens: int = 0, first_live: int = 0) -> None:
        self.pages: List[int] = list(pages or [])
        self.num_tokens = int(num_tokens)
        self.first_live = int(first_live)      # pages before this index have been given back

    def live_pages(self) -> List[int]:
        return [p for p in self.pages[self.first_live:] if p != NO_PAGE]
