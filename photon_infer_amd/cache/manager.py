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

The manager is host-side bookkeeping only; it never touches device memory.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..errors import CacheError, OutOfPagesError
from .pages import PagePool


@dataclass
class _Group:
    window: Optional[int]
    pool: PagePool
    table: np.ndarray                      # [max_slots, max_blocks] int32, -1 = no page
    next_block: list                       # [max_slots] blocks ever allocated (index of the next one)
    first_block: list                      # [max_slots] first block still held


@dataclass
class _Request:
    slot: int
    length: int = 0     # tokens whose keys are in the cache
    reserved: int = 0   # tokens that pages are held for (>= length)


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
        self.groups: List[_Group] = [
            _Group(w, PagePool(n), np.full((self.max_slots, self.max_blocks), -1, np.int32),
                   [0] * self.max_slots, [0] * self.max_slots)
            for w, n in zip(windows, counts)
        ]
        self._requests: Dict[Hashable, _Request] = {}
        self._free_slots: List[int] = list(range(self.max_slots - 1, -1, -1))

    # ------------------------------------------------------------------ queries
    def __contains__(self, rid: Hashable) -> bool:
        return rid in self._requests

    @property
    def num_live(self) -> int:
        return len(self._requests)

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_free

    def _req(self, rid: Hashable) -> _Request:
        try:
            return self._requests[rid]
        except KeyError:
            raise CacheError(f"request {rid!r} is not live in the cache") from None

    def slot(self, rid: Hashable) -> int:
        return self._req(rid).slot

    def length(self, rid: Hashable) -> int:
        return self._req(rid).length

    def pages_needed(self, rid: Optional[Hashable], new_tokens: int) -> List[int]:
        """Pages each group must still hand out for ``rid`` to grow by ``new_tokens``
        (``rid`` None: a request that is not admitted yet)."""
        r = self._requests.get(rid) if rid is not None else None
        target = (r.length if r else 0) + new_tokens
        blocks = -(-target // self.page_size)
        if r is None:
            return [blocks] * len(self.groups)
        slot = r.slot
        return [max(0, blocks - g.next_block[slot]) for g in self.groups]

    def can_reserve(self, rid: Optional[Hashable], new_tokens: int, held_back: Sequence[int] | None = None) -> bool:
        """Whether ``reserve`` would succeed; ``held_back[g]`` pages of group g count as taken."""
        need = self.pages_needed(rid, new_tokens)
        return all(n <= g.pool.num_free - (held_back[i] if held_back else 0)
                   for i, (n, g) in enumerate(zip(need, self.groups)))

    # ------------------------------------------------------------------ life cycle
    def admit(self, rid: Hashable) -> int:
        """Give ``rid`` a slot.  Its block-table rows start empty."""
        if rid in self._requests:
            raise CacheError(f"request {rid!r} is already live in the cache")
        if not self._free_slots:
            raise CacheError(f"no free slot: {self.max_slots} requests are live")
        slot = self._free_slots.pop()
        self._requests[rid] = _Request(slot)
        return slot

    def reserve(self, rid: Hashable, new_tokens: int) -> None:
        """Hold pages for positions ``length .. length + new_tokens - 1`` in every group,
        all or nothing (OutOfPagesError leaves everything as it was)."""
        r = self._req(rid)
        if new_tokens < 0:
            raise CacheError(f"cannot reserve {new_tokens} tokens")
        target = r.length + new_tokens
        if target > self.max_model_len:
            raise CacheError(f"request {rid!r} would hold {target} tokens; the limit is {self.max_model_len}")
        need = self.pages_needed(rid, new_tokens)
        for i, (n, g) in enumerate(zip(need, self.groups)):
            if n > g.pool.num_free:
                raise OutOfPagesError(
                    f"request {rid!r} needs {n} more pages in cache group {i}, {g.pool.num_free} are free")
        for n, g in zip(need, self.groups):
            if n:
                pages = g.pool.allocate(n)
                b = int(g.next_block[r.slot])
                g.table[r.slot, b:b + n] = pages
                g.next_block[r.slot] = b + n
        r.reserved = max(r.reserved, target)

    def commit(self, rid: Hashable, new_tokens: int) -> None:
        """The step wrote ``new_tokens`` more keys: advance the length and give back the
        pages that every window has passed."""
        r = self._req(rid)
        if r.length + new_tokens > r.reserved:
            raise CacheError(
                f"request {rid!r}: committing to {r.length + new_tokens} tokens but pages are held for {r.reserved}")
        r.length += new_tokens
        for g in self.groups:
            if g.window is None:
                continue
            # the next query sits at position >= length and reads keys >= length - window + 1
            first_needed = max(0, r.length - g.window + 1) // self.page_size
            lo = int(g.first_block[r.slot])
            hi = min(first_needed, int(g.next_block[r.slot]))
            if hi > lo:
                g.pool.free(int(p) for p in g.table[r.slot, lo:hi])
                g.table[r.slot, lo:hi] = -1
                g.first_block[r.slot] = hi

    def release(self, rid: Hashable) -> int:
        """The request ended (or was preempted): give back its pages and its slot."""
        r = self._req(rid)
        for g in self.groups:
            lo, hi = int(g.first_block[r.slot]), int(g.next_block[r.slot])
            if hi > lo:
                g.pool.free(int(p) for p in g.table[r.slot, lo:hi])
            g.table[r.slot, :] = -1
            g.next_block[r.slot] = 0
            g.first_block[r.slot] = 0
        del self._requests[rid]
        self._free_slots.append(r.slot)
        return r.slot

    def reset(self) -> None:
        for rid in list(self._requests):
            self.release(rid)

    # ------------------------------------------------------------------ for the step function
    def table_rows(self, group: int, slots: Sequence[int], width: Optional[int] = None) -> np.ndarray:
        """Block-table rows of ``slots`` (int32 [len(slots), width])."""
        g = self.groups[group]
        w = self.max_blocks if width is None else width
        return g.table[np.asarray(slots, dtype=np.int64), :w]

    def blocks_in_use(self, slots: Sequence[int]) -> int:
        """Largest block index + 1 among ``slots`` over all groups."""
        if not len(slots):
            return 0
        idx = np.asarray(slots, dtype=np.int64)
        return max(max(g.next_block[int(i)] for i in idx) for g in self.groups) if self.groups else 0

    # ------------------------------------------------------------------ checks and numbers
    def check_invariants(self) -> None:
        """No page lost, none held twice: every allocated page appears exactly once in the
        tables of live requests and every page in a table is allocated."""
        live_slots = {r.slot for r in self._requests.values()}
        if len(live_slots) != len(self._requests) or live_slots & set(self._free_slots):
            raise CacheError("slot bookkeeping is inconsistent")
        if len(live_slots) + len(self._free_slots) != self.max_slots:
            raise CacheError("a slot was lost")
        for gi, g in enumerate(self.groups):
            held: List[int] = []
            for s in range(self.max_slots):
                row = g.table[s]
                pages = row[row >= 0]
                if s not in live_slots and len(pages):
                    raise CacheError(f"group {gi}: free slot {s} still holds pages")
                lo, hi = int(g.first_block[s]), int(g.next_block[s])
                if len(pages) != hi - lo or (hi > lo and (row[lo:hi] < 0).any()):
                    raise CacheError(f"group {gi}: slot {s} table does not match its block range")
                held += [int(p) for p in pages]
            if len(held) != len(set(held)):
                raise CacheError(f"group {gi}: a page is held twice")
            if len(held) != g.pool.num_allocated or any(not g.pool.is_allocated(p) for p in held):
                raise CacheError(f"group {gi}: {g.pool.num_allocated} pages allocated but {len(held)} in tables")

    def utilization(self, group: int = 0) -> float:
        g = self.groups[group]
        return g.pool.num_allocated / g.pool.num_pages
