"""Fixed-size pages and their free list.

Reference: src/runtime/block_manager.cpp:14-141 - a LIFO stack of free block ids, an
``allocated`` bitmap that detects double frees and ids out of range, and all-or-nothing
allocation of several blocks.  LIFO order means a page that was just given back is the
next one handed out.

The bookkeeping itself is native (``csrc/runtime/cache.cpp``); this class is its handle.
"""
from __future__ import annotations

from typing import Iterable, List

from ..errors import CacheError, OutOfPagesError
from . import _native


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._lib = _native.lib()
        self._h = self._lib.pi_pool_create(self.num_pages)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.pi_pool_destroy(h)

    def _fail(self, status: int):
        msg = self._lib.pi_pool_error(self._h).decode()
        raise (OutOfPagesError if status == _native.OUT_OF_PAGES else CacheError)(msg)

    @property
    def num_free(self) -> int:
        return self._lib.pi_pool_num_free(self._h)

    @property
    def num_allocated(self) -> int:
        return self.num_pages - self.num_free

    def is_allocated(self, page: int) -> bool:
        return bool(self._lib.pi_pool_is_allocated(self._h, int(page)))

    def allocate(self, n: int = 1) -> List[int]:
        """``n`` pages or none: raises OutOfPagesError without taking any."""
        out = _native.int_array([0] * max(0, n))
        status = self._lib.pi_pool_allocate(self._h, int(n), out)
        if status:
            self._fail(status)
        return list(out[:n])

    def free(self, pages: Iterable[int]) -> None:
        pages = [int(p) for p in pages]
        status = self._lib.pi_pool_free(self._h, _native.int_array(pages), len(pages))
        if status:
            self._fail(status)

    def reset(self) -> None:
        self._lib.pi_pool_reset(self._h)
