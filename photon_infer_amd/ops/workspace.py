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
from typing import Dict, Optional, Tuple

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


def stream_layout_takes(w: torch.Tensor) -> bool:
    """Whether ``stream_layout`` has a form for ``w``."""
    return (w.dim() == 2 and w.dtype == torch.bfloat16 and w.is_contiguous() and w.shape[0] > 0 and w.shape[0] % 16 == 0
            and w.shape[1] > 0 and w.shape[1] % 64 == 0)


def stream_layout(w: torch.Tensor) -> Optional[torch.Tensor]:
    """The bfloat16 matrix ``w`` [N, K] (N a multiple of 16, K of 64, rows contiguous) as
    [N / 16][K / 64][2][4][16][8]: for every 16 rows and 64 columns, the 1 KB that a wave of the
    weight-streaming kernels loads with one instruction lies in a row (lane group g of a wave
    holds columns 16 g + 8 h .. + 7 of its row in its fragment h).  None for other matrices."""
    if not stream_layout_takes(w):
        return None
    N, K = w.shape
    tiles = w.view(N // 16, 16, K // 64, 4, 2, 8)          # [row block, row, k block, lane group, fragment, 8 columns]
    return tiles.permute(0, 2, 4, 3, 1, 5).contiguous().view(N, K)


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
        # weight matrices that have a second copy in the order the weight-streaming kernels read
        # (steps of up to 128 tokens): address of the matrix -> (copy, rows, columns, the matrix
        # itself: while it is kept here, nothing else can come to lie at its address)
        self.stream_copies: Dict[int, Tuple[torch.Tensor, int, int, torch.Tensor]] = {}

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

    def add_stream_copy(self, w: torch.Tensor) -> bool:
        """Keep a copy of the bfloat16 matrix ``w`` [N, K] in the weight-streaming kernels' order
        (``stream_layout``); products of up to 128 tokens with ``w`` then read the copy.  False,
        and nothing kept, for a matrix whose sizes the layout does not take."""
        copy = stream_layout(w)
        if copy is None:
            return False
        self.stream_copies[w.data_ptr()] = (copy, w.shape[0], w.shape[1], w)
        return True

    def drop_stream_copies(self) -> None:
        """Forget every copy (their memory goes back to the allocator); products read the matrices
        themselves again.  For a caller that changes a weight matrix after load: a copy is made
        once and never refreshed."""
        self.stream_copies.clear()

    def stream_copy_of(self, w: torch.Tensor, N: int, K: int) -> Optional[torch.Tensor]:
        entry = self.stream_copies.get(w.data_ptr())
        if entry is None or entry[1] != N or entry[2] != K:
            return None
        return entry[0]

    def take_pending(self, x: torch.Tensor) -> Optional[Partials]:
        """The pieces still to be added to ``x``, if any; they are the caller's to add."""
        p = self.pending
        if p is not None and p.is_for(x):
            self.pending = None
            return p.pieces
        return None
