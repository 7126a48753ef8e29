"""Fixed-size pages and their free list.

Reference: src/runtime/block_manager.cpp:14-141 - a LIFO stack of free block ids, an
``allocated`` bitmap that detects double frees and ids out of range, and all-or-nothing
allocation of several blocks.  LIFO order means a page that was just given back is the
next one handed out.
"""
from __future__ import annotations

from typing import Iterable, List

from ..errors import CacheError, OutOfPagesError


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))  # pop() hands out 0 first
        self._allocated = bytearray(self.num_pages)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_allocated(self) -> int:
        return self.num_pages - len(self._free)

    def is_allocated(self, page: int) -> bool:
        return 0 <= page < self.num_pages and bool(self._allocated[page])

    def allocate(self, n: int = 1) -> List[int]:
        """``n`` pages or none: raises OutOfPagesError without taking any."""
        if n < 0:
            raise CacheError(f"cannot allocate {n} pages")
        if n > len(self._free):
            raise OutOfPagesError(f"{n} pages asked for, {len(self._free)} of {self.num_pages} free")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._allocated[p] = 1
        return pages

    def free(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        seen = set()
        for p in pages:  # check all before changing anything
            if not 0 <= p < self.num_pages:
                raise CacheError(f"page id {p} is outside the pool of {self.num_pages}")
            if not self._allocated[p] or p in seen:
                raise CacheError(f"page {p} is freed twice")
            seen.add(p)
        for p in pages:
            self._allocated[p] = 0
            self._free.append(p)

    def reset(self) -> None:
        self._free = list(range(self.num_pages - 1, -1, -1))
        self._allocated = bytearray(self.num_pages)
