"""The cache manager: pages with a block table per request, in groups, plus state slots.

Reference: src/runtime/kv_cache_manager.cpp (one pool, same block id in all layers,
``allocate_sequence / extend_sequence / free_sequence``) and src/runtime/block_table.cpp
(request -> list of block ids, padded with -1 for the device).  Differences, all ours:

* layers whose mixers keep different things (all keys; the last W keys) form *groups*,
  each with a pool and block tables of its own;
* pages are taken on demand, one step at a time (the reference reserves a request's
  whole lifetime up front, include/photon/scheduler/continuous_batch_engine.hpp:98-103);
* a group with a window gives a page back as soon as every position in it is out of
  reach of all later queries;
* every live request owns a *slot*: the row of its block tables and the index of its
  fixed-size state, if any mixer keeps one.

The manager is host-side bookkeeping only; it never touches device memory.  The bookkeeping
itself is native (``csrc/runtime/cache.cpp``): this class maps request ids to slots, turns
status codes into exceptions, and hands out numpy views of the native block tables.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..errors import CacheError, OutOfPagesError
from . import _native


class _GroupPool:
    """What callers may ask about a group's page pool."""

    def __init__(self, manager: "CacheManager", index: int, num_pages: int):
        self._m, self._g, self.num_pages = manager, index, num_pages

    @property
    def num_free(self) -> int:
        return self._m._lib.pi_cache_free_pages(self._m._h, self._g)

    @property
    def num_allocated(self) -> int:
        return self.num_pages - self.num_free

    def is_allocated(self, page: int) -> bool:
        return bool(self._m._lib.pi_cache_page_allocated(self._m._h, self._g, int(page)))


class _Group:
    """A view of one cache group: its window, pool and block tables (numpy views of native memory)."""

    def __init__(self, manager: "CacheManager", index: int, window: Optional[int], num_pages: int):
        lib, h = manager._lib, manager._h
        self.window = window
        self.pool = _GroupPool(manager, index, num_pages)
        shape = (manager.max_slots, manager.max_blocks)
        self.table = np.ctypeslib.as_array(lib.pi_cache_table(h, index), shape=shape)          # -1 = no page
        self.next_block = np.ctypeslib.as_array(lib.pi_cache_next_block(h, index), shape=(manager.max_slots,))
        self.first_block = np.ctypeslib.as_array(lib.pi_cache_first_block(h, index), shape=(manager.max_slots,))


class CacheManager:
    def __init__(self, windows: Sequence[Optional[int]], page_size: int, num_pages: int | Sequence[int],
                 max_slots: int, max_model_len: int):
        """``windows``: one entry per cache group (None = keep all keys).
        ``num_pages``: pages of each group's pool (one number = the same for all)."""
        if page_size <= 0 or max_slots <= 0 or max_model_len <= 0:
            raise CacheError("page_size, max_slots and max_model_len must be positive")
        self.page_size = int(page_size)
        self.max_slots = int(max_slots)
        self.max_model_len = int(max_model_len)
        self.max_blocks = -(-self.max_model_len // self.page_size)
        counts = [num_pages] * len(windows) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(windows):
            raise CacheError(f"{len(windows)} cache groups but {len(counts)} pool sizes")
        if any(int(n) <= 0 for n in counts):
            raise CacheError(f"a page pool needs at least one page, got {counts}")
        self._lib = _native.lib()
        self._h = self._lib.pi_cache_create(len(windows), _native.int_array(-1 if w is None else int(w) for w in windows),
                                            self.page_size, _native.int_array(int(n) for n in counts), self.max_slots,
                                            self.max_model_len)
        if not self._h:
            raise CacheError("the native cache manager refused its sizes")
        self.groups: List[_Group] = [_Group(self, i, w, int(n)) for i, (w, n) in enumerate(zip(windows, counts))]
        self._lengths = np.ctypeslib.as_array(self._lib.pi_cache_lengths(self._h), shape=(self.max_slots,))
        self._slots: Dict[Hashable, int] = {}
        self._need = _native.int_array([0] * len(self.groups))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self.groups = []          # the views point into native memory
            self._lib.pi_cache_destroy(h)

    def _fail(self, status: int, rid: Hashable = None):
        msg = self._lib.pi_cache_error(self._h).decode()
        if rid is not None:
            msg = f"request {rid!r}: {msg}"
        raise (OutOfPagesError if status == _native.OUT_OF_PAGES else CacheError)(msg)

    # ------------------------------------------------------------------ queries
    def __contains__(self, rid: Hashable) -> bool:
        return rid in self._slots

    @property
    def num_live(self) -> int:
        return len(self._slots)

    @property
    def free_slots(self) -> int:
        return self._lib.pi_cache_free_slots(self._h)

    def free_pages(self, group: int = 0) -> int:
        return self._lib.pi_cache_free_pages(self._h, group)

    def slot(self, rid: Hashable) -> int:
        try:
            return self._slots[rid]
        except KeyError:
            raise CacheError(f"request {rid!r} is not live in the cache") from None

    def length(self, rid: Hashable) -> int:
        return int(self._lengths[self.slot(rid)])

    def pages_needed(self, rid: Optional[Hashable], new_tokens: int) -> List[int]:
        """Pages each group must still hand out for ``rid`` to grow by ``new_tokens``
        (``rid`` None or unknown: a request that is not admitted yet)."""
        slot = self._slots.get(rid, -1) if rid is not None else -1
        self._lib.pi_cache_pages_needed(self._h, slot, int(new_tokens), self._need)
        return list(self._need[:len(self.groups)])

    def can_reserve(self, rid: Optional[Hashable], new_tokens: int, held_back: Sequence[int] | None = None) -> bool:
        """Whether ``reserve`` would succeed; ``held_back[g]`` pages of group g count as taken."""
        slot = self._slots.get(rid, -1) if rid is not None else -1
        held = _native.int_array(held_back) if held_back else None
        return bool(self._lib.pi_cache_can_reserve(self._h, slot, int(new_tokens), held))

    # ------------------------------------------------------------------ life cycle
    def admit(self, rid: Hashable) -> int:
        """Give ``rid`` a slot.  Its block-table rows start empty."""
        if rid in self._slots:
            raise CacheError(f"request {rid!r} is already live in the cache")
        slot = self._lib.pi_cache_admit(self._h)
        if slot < 0:
            self._fail(_native.MISUSE)
        self._slots[rid] = slot
        return slot

    def reserve(self, rid: Hashable, new_tokens: int) -> None:
        """Hold pages for positions ``length .. length + new_tokens - 1`` in every group,
        all or nothing (OutOfPagesError leaves everything as it was)."""
        status = self._lib.pi_cache_reserve(self._h, self.slot(rid), int(new_tokens))
        if status:
            self._fail(status, rid)

    def commit(self, rid: Hashable, new_tokens: int) -> None:
        """The step wrote ``new_tokens`` more keys: advance the length and give back the
        pages that every window has passed."""
        status = self._lib.pi_cache_commit(self._h, self.slot(rid), int(new_tokens))
        if status:
            self._fail(status, rid)

    def pages_needed_step(self, rids: Sequence[Hashable], new_tokens: Sequence[int]) -> List[int]:
        """Pages each group must hand out for all of ``rids`` (live requests) to grow by their
        ``new_tokens`` in one step."""
        slots = [self._slots[r] for r in rids]
        status = self._lib.pi_cache_pages_needed_many(self._h, _native.int_array(slots), _native.int_array(new_tokens),
                                                      len(slots), self._need)
        if status:
            self._fail(status)
        return list(self._need[:len(self.groups)])

    def reserve_step(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """Pages for a whole step, all or nothing: either every request of the step can grow
        or nothing is taken (OutOfPagesError)."""
        n = len(slots)
        status = self._lib.pi_cache_reserve_many(self._h, _native.int_array(slots), _native.int_array(new_tokens), n)
        if status:
            self._fail(status)

    def commit_step(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        status = self._lib.pi_cache_commit_many(self._h, _native.int_array(slots), _native.int_array(new_tokens), len(slots))
        if status:
            self._fail(status)

    def release(self, rid: Hashable) -> int:
        """The request ended (or was preempted): give back its pages and its slot."""
        slot = self.slot(rid)
        status = self._lib.pi_cache_release(self._h, slot)
        if status:
            self._fail(status, rid)
        del self._slots[rid]
        return slot

    def reset(self) -> None:
        for rid in list(self._slots):
            self.release(rid)

    # ------------------------------------------------------------------ for the step function
    def table_rows(self, group: int, slots: Sequence[int], width: Optional[int] = None) -> np.ndarray:
        """Block-table rows of ``slots`` (int32 [len(slots), width], a copy)."""
        g = self.groups[group]
        w = self.max_blocks if width is None else width
        return g.table[np.asarray(slots, dtype=np.int64), :w]

    def lengths_of(self, slots: Sequence[int]) -> np.ndarray:
        """Cached tokens of ``slots`` (int32, a copy)."""
        return self._lengths[np.asarray(slots, dtype=np.int64)]

    def blocks_in_use(self, slots: Sequence[int]) -> int:
        """Largest block index + 1 among ``slots`` over all groups."""
        if not len(slots) or not self.groups:
            return 0
        idx = np.asarray(slots, dtype=np.int64)
        return int(max(g.next_block[idx].max() for g in self.groups))

    # ------------------------------------------------------------------ checks and numbers
    def check_invariants(self) -> None:
        """No page lost, none held twice: every allocated page appears exactly once in the
        tables of live requests and every page in a table is allocated."""
        if len(set(self._slots.values())) != len(self._slots) or len(self._slots) + self.free_slots != self.max_slots:
            raise CacheError("slot bookkeeping is inconsistent")
        status = self._lib.pi_cache_check(self._h)
        if status:
            self._fail(status)

    def utilization(self, group: int = 0) -> float:
        g = self.groups[group]
        return g.pool.num_allocated / g.pool.num_pages
