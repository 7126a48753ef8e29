"""Dispatch to the bfloat16 matrix-core kernels (module "bf16").

Each function returns True when it ran the operation and False when the sizes are not
ones its kernels take, in which case the caller uses the general kernel.

Which kernel takes what:
  * matrix products: K and the row strides multiples of 8, 16-byte aligned operands;
    up to 128 rows go to the weight-streaming kernels (k split over blocks where the output
    is narrow), more rows to the tile kernels;
  * attention: pages of a multiple of 16 tokens; a batch of single tokens with at most 16 heads
    per kv head goes to the key-split decode kernel (head_dim a multiple of 16 up to 256; for
    64 and 128 straight from the q|k|v projection), any other batch to the tile kernel
    (head_dim a multiple of 16 up to 256), its single tokens to the decode kernel.
"""
from __future__ import annotations

import ctypes
import functools
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import KernelError
from . import _lib
from .workspace import GEMM_PART_FLOATS, KernelWorkspace, KeyRanges, Partials, PendingUpdate

EPI_BF16, EPI_F32, EPI_ACCUM, EPI_SWIGLU = 0, 1, 2, 3
SKINNY_MAX_ROWS = 128          # up to this many tokens the weight-streaming kernels serve a product (measured against the tile kernel)
ROWS_PER_BLOCK = 32            # weight rows per block of the skinny kernel
BLOCKS_PER_UNIT = 2            # blocks of it wanted per compute unit to keep HBM busy (measured: 512 on 256 units; 384 and 768 are slower)
SHARED_FROM_TOKENS = 32        # more tokens than this: the skinny kernel that shares activations per block ...
SHARED_ROWS_PER_BLOCK = 64     # ... with this many weight rows per block ...
SHARED_BLOCKS_PER_UNIT = 1     # ... and one block wanted per compute unit
TILE_MAX_SPLITS = 4
BIG_TILES_PER_UNIT = 0.75      # 256 x 256 tiles (times k pieces) per compute unit from which the large-tile kernel is taken (the library's rule)
DEFAULT_UNITS = 256            # compute units assumed where no device can be asked (an MI355X)
BIG_MIN_K = 1024               # a piece of the large-tile kernel keeps at least this much of k
BIG_SPLIT_MIN_K = 6144         # ... and k is cut for it only from this length on
PIECES_BELOW_TILES = 200       # fewer 128 x 128 tiles than this: q, k, v of a prompt portion are left in k pieces too
TILE_HEAD_DIMS = tuple(range(16, 257, 16))         # head sizes of the prompt-attention tile kernel (above 128: rounds of 64 keys, 16 columns per wave)
DECODE_HEAD_DIMS = tuple(range(16, 257, 16))       # head sizes of the key-split decode kernel
FUSED_DECODE_HEAD_DIMS = (64, 128)                 # ... and of its form that starts from the q|k|v projection (whole halves of a head per fragment)
MAX_DECODE_SPLITS = 64         # the combine kernel holds one key range per lane
DECODE_WAVES_PER_UNIT = 2      # waves of the decode attention kernel per compute unit that fill the chip (measured at batch 1 to 64: more is never faster)
DECODE_MIN_KEYS_PER_SPLIT = 128


def _stream() -> int:
    return _lib.current_stream()


@functools.lru_cache(maxsize=None)
def _units_of(index: int) -> int:
    return int(torch.cuda.get_device_properties(index).multi_processor_count)


def compute_units() -> int:
    """Compute units of the current device: the split rules below count blocks and waves in
    multiples of it (256 on an MI355X, where they were measured)."""
    try:
        return _units_of(torch.cuda.current_device())
    except Exception:                    # no device in this process (rules asked for on the host)
        return DEFAULT_UNITS


def _gemm_ok(a, w, K, lda, ldw) -> bool:
    return K % 8 == 0 and lda % 8 == 0 and ldw % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0


def _skinny_splits(M: int, N: int, K: int) -> int:
    units = compute_units()
    if M > SHARED_FROM_TOKENS:     # the kernel that shares an activation tile per block: one block per compute unit
        groups, wanted = -(-N // SHARED_ROWS_PER_BLOCK), SHARED_BLOCKS_PER_UNIT * units
    else:
        groups, wanted = -(-N // ROWS_PER_BLOCK), BLOCKS_PER_UNIT * units
    splits = max(1, min(-(-wanted // groups), K // 256))
    while splits > 1 and splits * M * N > GEMM_PART_FLOATS:
        splits -= 1
    return splits


def _tile_splits(M: int, N: int, K: int) -> int:
    """k-split of the tile kernels: only when the output has too few tiles to fill the chip."""
    big = -(-M // 256) * -(-N // 256)
    units = compute_units()
    if K % 64 == 0:
        # a long k over few 256 x 256 tiles (the down projection of a 2,048-token prompt): as many
        # pieces on the large-tile kernel as give every compute unit one block (measured at
        # 2048 x 2048 x 8192: four pieces 72 us, against 87 us for two pieces on the small tiles,
        # and 6 us more in the norm that adds them)
        # and k long enough that the faster kernel outweighs the pieces' way through memory: the
        # o projection of such a prompt (k = 3,072 / 4,096, two pieces) took 68 / 93 us with its
        # norm against 61 / 86 us unsplit on the small tiles
        for pieces in (4, 3, 2):
            if (BIG_TILES_PER_UNIT * units <= big * pieces <= units and K >= max(pieces * BIG_MIN_K, BIG_SPLIT_MIN_K)
                    and pieces * M * N <= GEMM_PART_FLOATS):
                return pieces
    tiles = -(-M // 128) * -(-N // 128)
    splits = min(TILE_MAX_SPLITS, BLOCKS_PER_UNIT * units // max(1, tiles), K // 512)
    while splits > 1 and splits * M * N > GEMM_PART_FLOATS:
        splits -= 1
    return max(1, splits)


def flush(ws: Optional[KernelWorkspace]) -> None:
    """The product scratch is about to be reused: apply the update that still lives in it."""
    if ws is None or ws.pending is None:
        return
    p, ws.pending = ws.pending, None
    reduce_into(p.target, p.pieces, accumulate=True)
    ws.counts["flushed"] += 1


def _piece_buffer(ws: Optional[KernelWorkspace], floats: int, device) -> torch.Tensor:
    """Where the pieces of a split product go: the workspace's buffer (whose last tenant is
    applied first), or memory of this call's own."""
    if ws is None:
        return torch.empty(floats, dtype=torch.float32, device=device)
    if floats > GEMM_PART_FLOATS:
        # the split rules never ask for more; a kernel writing pieces past the buffer would fault the GPU
        raise KernelError(f"pieces of a split product need {floats} floats, the workspace holds {GEMM_PART_FLOATS}")
    flush(ws)
    return ws.gemm_part


def _streamed(ws: Optional[KernelWorkspace], w, N: int, K: int, ldw: int):
    """(address, tiled) of the weight matrix for the weight-streaming kernels: its copy in their
    own order when the workspace keeps one, else the matrix itself."""
    if ws is not None and ws.stream_copies and ldw == K:
        copy = ws.stream_copy_of(w, N, K)
        if copy is not None:
            return copy.data_ptr(), 1
    return w.data_ptr(), 0


def _skinny(out_ptr: int, epilogue: int, ldc: int, a, w, M, N, K, lda, ldw, splits: int,
            ws: Optional[KernelWorkspace], pieces_ws: bool = True) -> Optional[Partials]:
    """Run the weight-streaming kernel; returns the pieces when the product was split.
    ``pieces_ws`` False: the workspace is only asked for the weights' streaming copy."""
    buf = _piece_buffer(ws if pieces_ws else None, splits * M * N, a.device) if splits > 1 else None
    made = ctypes.c_int(0)
    w_ptr, tiled = _streamed(ws, w, N, K, ldw)
    _lib.call("bf16", "pi_gemm_skinny", out_ptr, epilogue, ldc, a.data_ptr(), lda, w_ptr, ldw, M, N, K, splits,
              None if buf is None else buf.data_ptr(), 0 if buf is None else buf.numel(), ctypes.byref(made), tiled, _stream())
    if made.value > 1:
        if ws is not None:
            ws.counts["split_products"] += 1
        return Partials(buf, made.value, M, N)
    return None


def _tiles_in_pieces(a, w, M, N, K, lda, ldw, splits: int, ws: Optional[KernelWorkspace]) -> Optional[Partials]:
    """The tile kernel with its k-range split: float32 pieces, nothing else written."""
    buf = _piece_buffer(ws, splits * M * N, a.device)
    made = _lib.load("bf16").pi_gemm_mfma_pieces(K, splits)
    _lib.call("bf16", "pi_gemm_mfma", buf.data_ptr(), EPI_F32, N, a.data_ptr(), lda, w.data_ptr(), ldw, M, N, K, splits,
              _stream())
    if ws is not None:
        ws.counts["split_products"] += 1
    return Partials(buf, made, M, N)


def reduce_into(out: torch.Tensor, p: Partials, accumulate: bool) -> None:
    epilogue = EPI_ACCUM if accumulate else (EPI_BF16 if out.dtype == torch.bfloat16 else EPI_F32)
    _lib.call("bf16", "pi_splitk_reduce", out.data_ptr(), epilogue, out.stride(0), p.part.data_ptr(), p.splits, p.M, p.N,
              _stream())


def gemm(out, a, w, accumulate, M, N, K, lda, ldw, ldc, may_defer=False, ws: Optional[KernelWorkspace] = None) -> bool:
    if not _gemm_ok(a, w, K, lda, ldw):
        return False
    if accumulate:
        epilogue = EPI_ACCUM
    elif out.dtype == torch.bfloat16:
        epilogue = EPI_BF16
    elif out.dtype == torch.float32:
        epilogue = EPI_F32
    else:
        return False
    may_defer = may_defer and ws is not None      # pieces can only wait in a workspace that outlives the call
    if M > SKINNY_MAX_ROWS:
        # few output tiles, long k: split k so that every compute unit has work; the pieces
        # stay in the workspace for the next norm of this stream
        splits = _tile_splits(M, N, K) if may_defer else 1
        if splits > 1:
            ws.pending = PendingUpdate(out, _tiles_in_pieces(a, w, M, N, K, lda, ldw, splits, ws))
            ws.counts["deferred"] += 1
            return True
        _lib.call("bf16", "pi_gemm_mfma", out.data_ptr(), epilogue, ldc, a.data_ptr(), lda, w.data_ptr(), ldw, M, N, K, 1,
                  _stream())
        return True
    pieces = _skinny(out.data_ptr(), epilogue, ldc, a, w, M, N, K, lda, ldw, _skinny_splits(M, N, K), ws)
    if pieces is not None:
        if may_defer:
            ws.pending = PendingUpdate(out, pieces)          # the next norm of this stream adds them
            ws.counts["deferred"] += 1
        else:
            _lib.call("bf16", "pi_splitk_reduce", out.data_ptr(), epilogue, ldc, pieces.part.data_ptr(), pieces.splits,
                      M, N, _stream())
    return True


RANGES_MAX_TOKENS = 16      # the weight-streaming kernel merges key ranges on the way in for up to this many tokens
RANGES_HEAD_DIM_STEP = 64   # ... of heads whose size is a multiple of its k step
# ... and for weights up to this size: the merging kernel has 64 weight rows per block, half the
# blocks of the plain one, which a larger matrix needs to stream at full rate (measured, batch 1
# to 16 at context 4,096: 8.4 MB 1 to 3 % faster per step, 19 MB and 34 MB 2 to 6 % slower)
RANGES_MAX_WEIGHT_BYTES = 12 << 20


def ranges_product_ok(tokens: int, head_dim: int, weight_bytes: int = 0) -> bool:
    return tokens <= RANGES_MAX_TOKENS and head_dim % RANGES_HEAD_DIM_STEP == 0 and weight_bytes <= RANGES_MAX_WEIGHT_BYTES


def merge_ranges(out: torch.Tensor, kr: KeyRanges) -> None:
    """The merged attention output, bfloat16 [tokens, heads * head_dim], by the merging kernel."""
    _lib.call("bf16", "pi_attention_combine_rows", out.data_ptr(), out.stride(0), kr.rows.data_ptr(), kr.tokens,
              kr.part.data_ptr(), kr.heads, kr.head_dim, kr.count, _stream())


def gemm_from_ranges(out, kr: KeyRanges, w, accumulate, N, ldw, ldc, may_defer, ws: Optional[KernelWorkspace]) -> bool:
    """out (+)= merged(kr) @ w^T by the weight-streaming kernel, which merges the key ranges as it
    stages its activations; the same bits as merging first."""
    M, K = kr.tokens, kr.heads * kr.head_dim
    if not ranges_product_ok(M, kr.head_dim, N * K * 2) or w.dtype != torch.bfloat16 or w.stride(1) != 1 or ldw % 8 or w.data_ptr() % 16:
        return False
    if accumulate:
        epilogue = EPI_ACCUM
    elif out.dtype == torch.bfloat16:
        epilogue = EPI_BF16
    elif out.dtype == torch.float32:
        epilogue = EPI_F32
    else:
        return False
    splits = _skinny_splits(M, N, K)
    buf = _piece_buffer(ws, splits * M * N, w.device) if splits > 1 else None
    made = ctypes.c_int(0)
    w_ptr, tiled = _streamed(ws, w, N, K, ldw)
    _lib.call("bf16", "pi_gemm_skinny_ranges", out.data_ptr(), epilogue, ldc, kr.part.data_ptr(), kr.heads, kr.head_dim, kr.count,
              w_ptr, ldw, M, N, splits, None if buf is None else buf.data_ptr(), 0 if buf is None else buf.numel(),
              ctypes.byref(made), tiled, _stream())
    if ws is not None:
        ws.counts["ranges_merged_by_product"] += 1
    if made.value > 1:
        pieces = Partials(buf, made.value, M, N)
        if ws is not None:
            ws.counts["split_products"] += 1
        if may_defer and ws is not None:
            ws.pending = PendingUpdate(out, pieces)
            ws.counts["deferred"] += 1
        else:
            _lib.call("bf16", "pi_splitk_reduce", out.data_ptr(), epilogue, ldc, pieces.part.data_ptr(), pieces.splits, M, N,
                      _stream())
    return True


def gemm_pieces(a, w, ws: Optional[KernelWorkspace]) -> Optional[Partials]:
    """a @ w^T left in pieces in the workspace, if this product is one whose k-range is split."""
    if ws is None:
        return None
    M, K = a.shape
    N = w.shape[0]
    lda, ldw = a.stride(0) if M > 1 else K, w.stride(0)
    if not _gemm_ok(a, w, K, lda, ldw) or a.stride(1) != 1 or w.stride(1) != 1:
        return None
    if M > SKINNY_MAX_ROWS:
        # a prompt portion of a few hundred tokens has too few 128 x 128 tiles for the chip:
        # split k there too, the consumer adds the pieces
        tiles = -(-M // 128) * -(-N // 128)
        splits = _tile_splits(M, N, K) if tiles < PIECES_BELOW_TILES else 1
        if splits <= 1:
            return None
        p = _tiles_in_pieces(a, w, M, N, K, lda, ldw, splits, ws)
        return p if p.splits > 1 else None
    splits = _skinny_splits(M, N, K)
    if splits <= 1:
        return None
    return _skinny(0, EPI_F32, N, a, w, M, N, K, lda, ldw, splits, ws)


def gemm_swiglu(out, a, w, M, N, K, lda, ldw, ws: Optional[KernelWorkspace] = None) -> bool:
    """``w`` [N = 2I, K] with gate / up rows interleaved in blocks of 16; out [M, I] bfloat16."""
    if not _gemm_ok(a, w, K, lda, ldw) or N % 32 or out.dtype != torch.bfloat16:
        return False
    if M > SKINNY_MAX_ROWS:
        _lib.call("bf16", "pi_gemm_mfma", out.data_ptr(), EPI_SWIGLU, out.stride(0), a.data_ptr(), lda, w.data_ptr(), ldw,
                  M, N, K, 1, _stream())
    else:
        _skinny(out.data_ptr(), EPI_SWIGLU, out.stride(0), a, w, M, N, K, lda, ldw, 1, ws, pieces_ws=False)
    return True


# ----------------------------------------------------------------------------- attention
def attention_tile_rows(num_heads: int, num_kv_heads: int, head_dim: int) -> int:
    return _lib.load("bf16").pi_attention_tile_rows(num_heads, num_kv_heads, head_dim)


def attention_blocks_per_unit(head_dim: int) -> int:
    """Blocks of the tile kernel that one compute unit holds at a time: two up to head size 64,
    one above (its LDS and registers).  More seats than that only queue behind the first and
    leave the deal of tiles to blocks uneven: at head size 128 a 2,048-token prompt took 104 us
    with two seats per unit and 84 us with one."""
    return 2 if head_dim <= 64 else 1


def deal_tiles(walks: List[int], seats: int) -> np.ndarray:
    """[rounds, seats] tile indices (-1: none): the tiles sorted by the keys they walk, longest
    first, dealt to ``seats`` blocks back and forth so that the blocks' sums come out close."""
    by_work = sorted(range(len(walks)), key=lambda i: -walks[i])
    rounds = -(-len(by_work) // seats)
    order = np.full((rounds, seats), -1, np.int32)
    for k in range(rounds):
        part = by_work[k * seats:(k + 1) * seats]
        cols = range(len(part)) if k % 2 == 0 else range(seats - 1, seats - 1 - len(part), -1)
        for c, t in zip(cols, part):
            order[k, c] = t
    return order


@dataclass(frozen=True)
class AttentionPlanner:
    """Makes a step's work lists for the prompt-attention tile kernel.  Mixers whose planners are
    equal (same tile height, window, kv heads) share one plan per step.  ``plan`` runs on the
    host before the step's metadata is uploaded; its arrays ride in that one copy."""

    tile_rows: int            # query rows of a tile (the kernel's, for these head counts)
    window: int               # 0: all keys
    num_kv_heads: int
    singles_apart: bool       # requests that bring one token go to the key-split kernel instead
    units: int                # compute units of the device
    blocks_per_unit: int = 2  # blocks that a unit holds at a time (attention_blocks_per_unit)

    def plan(self, q_lens: Sequence[int], kv_lens: Sequence[int]):
        """None for a step of single tokens only (the key-split kernel needs no list); otherwise
        (int32 host arrays by name, a function from their device views to a ``TilePlan``)."""
        if self.singles_apart and all(n == 1 for n in q_lens):
            return None
        tile_rows, window = self.tile_rows, self.window
        singles = tuple(r for r, n in enumerate(q_lens) if n == 1) if self.singles_apart else ()
        if len(singles) == len(q_lens):
            singles = ()
        skipped = set(singles)
        req, q0, walks, first_row, n_tok = [], [], [], [], []
        row0 = 0
        for r, (n, kv) in enumerate(zip(q_lens, kv_lens)):
            if r not in skipped:
                for start in range(0, n, tile_rows):
                    req.append(r)
                    q0.append(start)
                    first = kv - n + start                         # position of the tile's first token
                    last = first + min(tile_rows, n - start) - 1
                    lo = max(0, first - window + 1) if window > 0 else 0
                    walks.append(last // 128 - lo // 128 + 1)
                    first_row.append(row0 + start)
                    n_tok.append(min(tile_rows, n - start))
            row0 += n
        seats_wanted = max(1, self.blocks_per_unit * self.units // max(1, self.num_kv_heads))
        # too few tiles for the chip (a portion of a few hundred tokens): cut the key range of
        # the long ones into equal shares; the shares' partial results are merged afterwards
        cuts = cut_count(walks, seats_wanted)
        t_req, t_q0, t_cut, t_z0, t_walk, rows = [], [], [], [], [], []
        for i in range(len(req)):
            k = cuts if cuts > 1 and walks[i] >= 2 * cuts else 1
            z0 = len(rows) if k > 1 else 0
            if k > 1:
                rows.extend(range(first_row[i], first_row[i] + n_tok[i]))
            for c in range(k):
                t_req.append(req[i]); t_q0.append(q0[i]); t_cut.append(c | (k << 8)); t_z0.append(z0)
                t_walk.append(-(-walks[i] // k))
        seats = max(1, min(len(t_req), seats_wanted))
        order = deal_tiles(t_walk, seats)
        arrays = {"req": np.asarray(t_req, np.int32), "q0": np.asarray(t_q0, np.int32), "cut": np.asarray(t_cut, np.int32),
                  "z0": np.asarray(t_z0, np.int32), "rows": np.asarray(rows, np.int32), "order": order.reshape(-1),
                  "singles": np.asarray(singles, np.int32)}
        z, rounds = len(rows), order.shape[0]
        longest_single = max((kv_lens[r] for r in singles), default=0)

        def finish(views: Dict[str, torch.Tensor]) -> "TilePlan":
            return TilePlan(req=views["req"], q0=views["q0"], cut=views["cut"], z0=views["z0"], rows=views["rows"],
                            cut_tokens=z, cuts=cuts if z else 1, order=views["order"], rounds=rounds, seats=seats,
                            singles=singles, single_ids=views["singles"], longest_single=longest_single)

        return arrays, finish


@functools.lru_cache(maxsize=None)
def attention_planner(dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                      device) -> Optional[AttentionPlanner]:
    """The planner for a mixer of these sizes, or None when the general kernel serves it."""
    if dtype != torch.bfloat16 or head_dim not in TILE_HEAD_DIMS or page_size % 16:
        return None
    tile_rows = attention_tile_rows(num_heads, num_kv_heads, head_dim)
    if tile_rows < 1:
        return None
    units = torch.cuda.get_device_properties(device).multi_processor_count
    return AttentionPlanner(tile_rows, int(window), num_kv_heads, num_heads // num_kv_heads <= 16, units,
                            attention_blocks_per_unit(head_dim))


def upload_arrays(arrays: Dict[str, np.ndarray], device) -> Dict[str, torch.Tensor]:
    """Concatenate int32 arrays (each padded to 16 bytes), copy once, return device views."""
    offsets, total = {}, 0
    for name, arr in arrays.items():
        offsets[name] = (total, arr.size)
        total += (arr.size + 3) // 4 * 4
    packed = np.zeros(max(total, 4), np.int32)
    for name, arr in arrays.items():
        o, n = offsets[name]
        packed[o:o + n] = arr.reshape(-1)
    dev = torch.from_numpy(packed).to(device)
    return {name: dev[o:o + n] for name, (o, n) in offsets.items()}


def _tile_plan(ctx, planner: AttentionPlanner, device) -> "TilePlan":
    """The step's plan: the one the step function uploaded with its metadata, or - for a caller
    that made its context by hand - one made and uploaded here."""
    plans = getattr(ctx, "plans", None)
    if plans is None:
        plans = ctx.plans = {}
    plan = plans.get(planner)
    if plan is None:
        arrays, finish = planner.plan(ctx.q_lens, ctx.kv_lens)
        plan = plans[planner] = finish(upload_arrays(arrays, device))
    return plan


@dataclass
class TilePlan:
    """A step's work list for the tile kernel (device int32 arrays, one entry per tile or per
    share of a cut tile)."""

    req: torch.Tensor          # the entry's request
    q0: torch.Tensor           # its first token among the request's tokens of this step
    cut: torch.Tensor          # share | shares << 8 of the tile's key range
    z0: torch.Tensor           # first row of the tile in ``rows`` (cut tiles only)
    rows: torch.Tensor         # token rows of the cut tiles, in the order of their partial results
    cut_tokens: int
    cuts: int                  # shares per cut tile (the same for all of a step)
    order: torch.Tensor        # [rounds, seats]: which entry a block takes in which round (-1: none)
    rounds: int
    seats: int
    singles: Tuple[int, ...] = ()             # requests that bring one token beside requests that bring more
    single_ids: Optional[torch.Tensor] = None  # the same on the device
    longest_single: int = 0                   # the longest context among them


MAX_TILE_CUTS = 8
MIN_ROUNDS_PER_SHARE = 4       # a share of a cut tile walks at least this many rounds of 128 keys ...
MIN_ROUNDS_SAVED = 6           # ... and the cut shortens the longest walk by at least this many


def cut_count(walks: List[int], seats_wanted: int) -> int:
    """In how many shares the key range of a step's long tiles is cut: 1 unless the tiles are
    fewer than half the blocks the chip holds; then as many as fill it, while a share keeps
    enough rounds of 128 keys to be worth an entry of its own (its queries loaded again, its
    partial result written and merged: about the time of six rounds).  Measured at head sizes
    64 and 128, 64 to 1,024 tokens ending at 256 to 8,192: shares of two rounds made 256 tokens
    at 2,048 slower than uncut (56 us against 46; with shares of four 29 us), and two shares of
    a walk of eight rounds or less never paid."""
    tiles = len(walks)
    if tiles == 0 or tiles * 2 > seats_wanted:
        return 1
    longest = max(walks)
    cuts = min(MAX_TILE_CUTS, seats_wanted // tiles, longest // MIN_ROUNDS_PER_SHARE)
    if cuts < 2 or longest - -(-longest // cuts) < MIN_ROUNDS_SAVED:
        return 1
    return cuts


def decode_length_bucket(max_kv_len: int) -> int:
    """The power of two (at least one key range's worth) that a decode step's longest context
    is rounded up to.  Key ranges are chosen per bucket, so a step gives the same numbers
    whether it runs eagerly or replays the graph captured for its bucket."""
    bucket = DECODE_MIN_KEYS_PER_SPLIT
    while bucket < max_kv_len:
        bucket *= 2
    return bucket


def decode_splits(R: int, num_kv_heads: int, max_kv_len: int) -> int:
    """Key ranges per (request, kv head): enough waves to fill the chip, no more than the
    keys of the step's length bucket are worth."""
    splits = max(1, min(MAX_DECODE_SPLITS, -(-DECODE_WAVES_PER_UNIT * compute_units() // (R * num_kv_heads))))
    return min(splits, max(1, decode_length_bucket(max_kv_len) // DECODE_MIN_KEYS_PER_SPLIT))


def _attn_part(ws: Optional[KernelWorkspace], floats: int, device) -> torch.Tensor:
    return ws.attn_part if ws is not None else torch.empty(max(4, floats), dtype=torch.float32, device=device)


def _decode_splits_that_fit(ws, n_req: int, num_heads: int, num_kv_heads: int, head_dim: int, longest: int) -> int:
    splits = decode_splits(n_req, num_kv_heads, longest)
    if ws is not None:
        while splits > 1 and n_req * num_heads * splits * (head_dim + 4) > ws.attn_part.numel():
            splits -= 1
    return splits


def paged_attention(out, q, k_cache, v_cache, block_table, ctx, num_heads, num_kv_heads, head_dim,
                    page_size, scale, window, pages, ws: Optional[KernelWorkspace] = None) -> bool:
    if head_dim not in DECODE_HEAD_DIMS or page_size % 16 or q.data_ptr() % 16 or q.stride(0) % 8 or out.stride(0) % 4:
        return False
    G = num_heads // num_kv_heads
    R = ctx.R

    def decode_kernel(n_req: int, req_ids: int, longest: int) -> None:
        splits = _decode_splits_that_fit(ws, n_req, num_heads, num_kv_heads, head_dim, longest)
        part = _attn_part(ws, n_req * num_heads * splits * (head_dim + 4), q.device)
        _lib.call("bf16", "pi_attention_decode", out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0),
                  k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
                  ctx.q_start.data_ptr(), ctx.kv_len.data_ptr(), req_ids, n_req, num_heads, num_kv_heads, head_dim,
                  page_size, float(scale), int(window), pages, splits, part.data_ptr(), part.numel(), _stream())

    if ctx.all_decode and G <= 16:
        decode_kernel(R, 0, ctx.max_kv_len)
        return True
    planner = attention_planner(q.dtype, num_heads, num_kv_heads, head_dim, page_size, window, q.device)
    if planner is None:
        return False
    # A step of prompt portions and single tokens: the single tokens, whose keys no other token
    # of the step shares, go to the key-split kernel (a tile of one token would walk its whole
    # context in one block, mostly on padding); the portions go to the tile kernel.
    plan = _tile_plan(ctx, planner, q.device)
    if plan.singles:
        decode_kernel(len(plan.singles), plan.single_ids.data_ptr(), plan.longest_single)
    floats = plan.cut_tokens * num_heads * plan.cuts * (head_dim + 4)
    tile_part = ws.tile_part_for(floats) if ws is not None else torch.empty(max(4, floats), dtype=torch.float32, device=q.device)
    _lib.call("bf16", "pi_attention_prefill_mfma", out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0),
              k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
              ctx.q_start.data_ptr(), ctx.kv_len.data_ptr(), plan.req.data_ptr(), plan.q0.data_ptr(), plan.cut.data_ptr(),
              plan.z0.data_ptr(), tile_part.data_ptr(), plan.order.data_ptr(), plan.rounds, plan.seats, num_heads,
              num_kv_heads, head_dim, page_size, float(scale), int(window), pages, _stream())
    if plan.cut_tokens:
        _lib.call("bf16", "pi_attention_combine_rows", out.data_ptr(), out.stride(0), plan.rows.data_ptr(), plan.cut_tokens,
                  tile_part.data_ptr(), num_heads, head_dim, plan.cuts, _stream())
    return True


def decode_attention_from_projection(out, qkv, ctx, table, num_heads, num_kv_heads, head_dim, k_cache, v_cache,
                                     block_table, page_size, scale, window, pages, write_kv,
                                     ws: Optional[KernelWorkspace] = None, leave_ranges: int = 0):
    """A step of single tokens: attention straight from the q|k|v projection (``qkv``: a bfloat16
    tensor [T, N] or ``Partials``), which the kernel rotates by ``table`` (the step's cos / sin
    table [T, head_dim], or None) and whose keys and values it stores.  False: not for these sizes.
    ``leave_ranges`` (0: never; else the bytes of the weight matrix that reads the output next):
    when the keys were split into ranges and that product can merge them (``ranges_product_ok``),
    they are returned as ``KeyRanges`` and ``out`` is left alone."""
    G = num_heads // num_kv_heads
    if not ctx.all_decode or G > 16 or head_dim not in FUSED_DECODE_HEAD_DIMS or page_size % 16 or out.stride(0) % 4:
        return False
    R = ctx.R
    pieces = isinstance(qkv, Partials)
    need = (num_heads + (2 * num_kv_heads if write_kv else 0)) * head_dim
    if (qkv.M if pieces else qkv.shape[0]) != R or (qkv.N if pieces else qkv.shape[1]) < need:
        return False
    if (qkv.N % 4 or qkv.part.data_ptr() % 16) if pieces else (qkv.stride(0) % 8 or qkv.stride(1) != 1 or qkv.data_ptr() % 16):
        return False
    splits = _decode_splits_that_fit(ws, R, num_heads, num_kv_heads, head_dim, ctx.max_kv_len)
    part = _attn_part(ws, R * num_heads * splits * (head_dim + 4), out.device)
    leave = leave_ranges > 0 and ws is not None and splits > 1 and ranges_product_ok(R, head_dim, leave_ranges)
    _lib.call("bf16", "pi_attention_decode_fused", out.data_ptr(), out.stride(0),
              None if pieces else qkv.data_ptr(), 0 if pieces else qkv.stride(0),
              qkv.part.data_ptr() if pieces else None, qkv.splits if pieces else 0, qkv.N if pieces else 0, R,
              None if table is None else table.data_ptr(), int(bool(write_kv)), k_cache.data_ptr(), v_cache.data_ptr(),
              block_table.data_ptr(), block_table.shape[1], ctx.q_start.data_ptr(), ctx.kv_len.data_ptr(), R, num_heads,
              num_kv_heads, head_dim, page_size, float(scale), int(window), pages, splits, part.data_ptr(),
              part.numel(), int(not leave), _stream())
    if leave:
        return KeyRanges(part, splits, R, num_heads, head_dim, ctx.q_start)
    return True
