"""Scratch memory of the kernels, owned by whoever runs steps (one per ``ModelRunner``).

Nothing in this package keeps kernel state of its own.  The pieces of a product that was split
over k, the partial results of attention split over keys and the chunk records of the sampling
kernels live in a ``KernelWorkspace``; so does the one update of a residual stream that may
still be in pieces (see ``ops.gemm(..., may_defer=True)``).  Two runners have two workspaces
and never see each other's pieces; an op called without a workspace takes what it needs from
torch's allocator for that call and leaves nothing pending.
"""
from __future__ import annotations

from collections import Counter
from dataclasses import dataclass
from typing import Optional

import torch

GEMM_PART_FLOATS = 16 << 20    # pieces of products split over k (64 MB)
ATTN_PART_FLOATS = 4 << 20     # key-split partial results of decode attention
SAMPLE_FLOATS = 1 << 18        # chunk records of the sampling kernels


@dataclass
class Partials:
    """A product [M, N] whose k-range was split: ``part`` holds float32 [splits, M, N]."""

    part: torch.Tensor
    splits: int
    M: int
    N: int


@dataclass
class KeyRanges:
    """The attention output of a decode step (token r is request r) whose key ranges are not
    merged yet: ``part`` holds float32 [tokens, heads, count, head_dim + 4] (a range's output not
    yet normalised, then its maximum and its sum of weights).  It lives in the workspace's
    attention buffer, so it has to be consumed (``ops.gemm`` takes it as its activations) before
    the next attention of that workspace runs.  ``rows``: int32 device array, row of each token."""

    part: torch.Tensor
    count: int
    tokens: int
    heads: int
    head_dim: int
    rows: torch.Tensor

    def __bool__(self) -> bool:
        return True


@dataclass
class PendingUpdate:
    """``target += sum(pieces)`` that has not been applied yet."""

    target: torch.Tensor
    pieces: Partials

    def is_for(self, x: torch.Tensor) -> bool:
        t = self.target
        return t is x or (t.data_ptr() == x.data_ptr() and t.shape == x.shape and t.stride() == x.stride())


class KernelWorkspace:
    """Buffers are made at first use and kept; ``counts`` says which paths a step took (tests
    read it: ``split_products``, ``deferred``, ``added_by_norm``, ``applied``, ``flushed``,
    ``discarded``, ``qkv_pieces``, ``ranges_merged_by_product``)."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._gemm_part: Optional[torch.Tensor] = None
        self._attn_part: Optional[torch.Tensor] = None
        self._tile_part: Optional[torch.Tensor] = None
        self._sample_part: Optional[torch.Tensor] = None
        self.pending: Optional[PendingUpdate] = None
        self.counts: Counter = Counter()

    def _buffer(self, name: str, floats: int) -> torch.Tensor:
        buf = getattr(self, name)
        if buf is None or buf.numel() < floats:
            buf = torch.empty(floats, dtype=torch.float32, device=self.device)
            setattr(self, name, buf)
        return buf

    @property
    def gemm_part(self) -> torch.Tensor:
        return self._buffer("_gemm_part", GEMM_PART_FLOATS)

    @property
    def attn_part(self) -> torch.Tensor:
        return self._buffer("_attn_part", ATTN_PART_FLOATS)

    @property
    def sample_part(self) -> torch.Tensor:
        return self._buffer("_sample_part", SAMPLE_FLOATS)

    def tile_part_for(self, floats: int) -> torch.Tensor:
        """Partial results of cut tiles, grown on demand."""
        return self._buffer("_tile_part", max(4, floats))

    def prepare(self, matrix_core_kernels: bool) -> None:
        """Make the buffers of fixed size now (before anything is captured into a graph)."""
        self.sample_part
        if matrix_core_kernels:
            self.gemm_part
            self.attn_part

    def take_pending(self, x: torch.Tensor) -> Optional[Partials]:
        """The pieces still to be added to ``x``, if any; they are the caller's to add."""
        p = self.pending
        if p is not None and p.is_for(x):
            self.pending = None
            return p.pieces
        return None
