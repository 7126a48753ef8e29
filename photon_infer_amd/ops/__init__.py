"""Python face of the HIP kernels: shape / dtype / device checks, then one C call.

Every function works on tensors that live on the GPU and launches on torch's current
stream.  There is no CPU path: a tensor on the CPU, or a kernel library that cannot
be built or loaded, is an error.

Dispatch rule: bfloat16 operands whose sizes the matrix-core kernels take go to those
kernels (module "bf16"); everything else - float32, mixed storage types, odd sizes -
goes to the general kernels (module "core"), which take any size.
``use_fast_kernels(False)`` forces the general kernels (tests compare the two).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..errors import KernelError
from . import _lib
from .workspace import KernelWorkspace, KeyRanges, Partials, stream_layout, stream_layout_takes

PI_F32, PI_BF16 = 0, 1
MAX_HEAD_DIM = 256

_FAST = True


def use_fast_kernels(enabled: bool) -> bool:
    """Switch the matrix-core kernels on or off; returns the previous setting."""
    global _FAST
    prev, _FAST = _FAST, bool(enabled)
    return prev


def fast_kernels_enabled() -> bool:
    return _FAST


def ensure_loaded(dtype: torch.dtype) -> None:
    """Build / load what a model of compute dtype ``dtype`` needs."""
    _lib.load("core")
    if dtype == torch.bfloat16 and _FAST and _lib.build.MODULES["bf16"]:
        _lib.load("bf16")


# ----------------------------------------------------------------------------- helpers
def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return PI_F32
    if t.dtype == torch.bfloat16:
        return PI_BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernels run on the GPU only; got a tensor on " + str(t.device))


def _stream() -> int:
    return _lib.current_stream()


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride (elements) of a 2-D tensor whose rows are dense."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what}: expected a 2-D tensor with dense rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what}: expected a contiguous int32 tensor, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what}: expected at least {n} entries, got {t.numel()}")


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Sizes the attention kernels take; anything else is refused here, by name."""
    if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
        raise KernelError(f"attention: {num_heads} heads is not a positive multiple of {num_kv_heads} kv heads")
    if head_dim <= 0 or head_dim % 16 or head_dim > MAX_HEAD_DIM:
        raise KernelError(f"attention: head_dim {head_dim} must be a multiple of 16 up to {MAX_HEAD_DIM}")


# ----------------------------------------------------------------------------- ops
def embedding(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> None:
    """out[t, :] = float32(table[ids[t], :])."""
    _gpu(out, table, ids)
    T, D = out.shape
    if out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embedding: output must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != D or not table.is_contiguous():
        raise KernelError(f"embedding: table shape {tuple(table.shape)} does not match width {D}")
    _i32(ids, "embedding ids", T)
    _lib.call("core", "pi_embedding", out.data_ptr(), table.data_ptr(), _dt(table), ids.data_ptr(), T, D,
              table.shape[0], _stream())


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None, ws: Optional[KernelWorkspace] = None) -> None:
    """out[m, :] = weight * x[r, :] / sqrt(mean(x[r, :]^2) + eps), r = rows[m] (or m).  An update of
    ``x`` that is still pending in ``ws`` is added first, in the same pass, and written back to
    ``x`` (with ``rows``: to those rows only; the others are not read again by this caller)."""
    _gpu(out, x, weight, rows)
    M, D = out.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or x.dim() != 2 or x.shape[1] != D:
        raise KernelError(f"rmsnorm: input must be contiguous float32 [*, {D}], got {x.dtype} {tuple(x.shape)}")
    if not out.is_contiguous() or weight.shape != (D,) or not weight.is_contiguous():
        raise KernelError(f"rmsnorm: output must be contiguous and weight [{D}], got weight {tuple(weight.shape)}")
    if rows is None:
        if x.shape[0] != M:
            raise KernelError(f"rmsnorm: {x.shape[0]} input rows for {M} output rows")
    else:
        _i32(rows, "rmsnorm rows", M)
    pending = ws.take_pending(x) if ws is not None else None
    if pending is not None:
        ws.counts["added_by_norm"] += 1
    part, splits = (pending.part.data_ptr(), pending.splits) if pending is not None else (None, 0)
    _lib.call("core", "pi_rmsnorm", out.data_ptr(), _dt(out), x.data_ptr(), _ptr(rows), weight.data_ptr(),
              _dt(weight), float(eps), M, D, part, splits, x.shape[0], _stream())


# ----------------------------------------------------------------------------- deferred updates
# A product into the residual stream whose k-range was split over blocks may stay in pieces
# (``Partials`` in the caller's ``KernelWorkspace``) until the next reader of the stream:
# ``rmsnorm`` folds the sum of the pieces and the residual add into its own pass.  Whoever reads
# the stream in any other way calls ``materialize`` first.  Only callers that pass
# ``may_defer=True`` and a workspace to ``gemm`` ever leave an update pending (one at most per
# workspace), and a block arrangement must materialize before it hands the stream to a part that
# does not read it through ``rmsnorm``.
def materialize(x: torch.Tensor, ws: Optional[KernelWorkspace]) -> torch.Tensor:
    """Apply an update of ``x`` that is still pending in ``ws``, if there is one."""
    p = ws.take_pending(x) if ws is not None else None
    if p is not None:
        from . import fast
        fast.reduce_into(x, p, accumulate=True)
        ws.counts["applied"] += 1
    return x


def reset_deferred(ws: Optional[KernelWorkspace]) -> None:
    """Forget a pending update (start of a step: nothing of an earlier, failed step may linger)."""
    if ws is not None:
        ws.pending = None


def discard_deferred(x: torch.Tensor, ws: Optional[KernelWorkspace]) -> None:
    """Forget a pending update of ``x`` (the stream is not read again)."""
    if ws is not None and ws.take_pending(x) is not None:
        ws.counts["discarded"] += 1


def swiglu(out: torch.Tensor, gate_up: torch.Tensor, block: int = 0) -> None:
    """out[t, i] = silu(gate) * up.  ``block`` = 0: gate in columns [0, I), up in [I, 2I);
    ``block`` = b: gate and up interleaved in blocks of b columns."""
    _gpu(out, gate_up)
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype or not (out.is_contiguous() and gate_up.is_contiguous()):
        raise KernelError(f"swiglu: expected gate_up [{T}, {2 * I}] of {out.dtype}, got {tuple(gate_up.shape)} {gate_up.dtype}")
    if block < 0 or (block and I % block):
        raise KernelError(f"swiglu: interleave block {block} does not divide {I}")
    _lib.call("core", "pi_swiglu", out.data_ptr(), gate_up.data_ptr(), _dt(out), T, I, int(block), _stream())


def gemm_swiglu(out: torch.Tensor, a: torch.Tensor, w_gate_up: torch.Tensor, block: int = 0,
                ws: Optional[KernelWorkspace] = None) -> None:
    """out[M, I] = silu(a @ Wg^T) * (a @ Wu^T) where ``w_gate_up`` [2I, K] holds the gate and
    up rows in halves (``block`` 0) or interleaved in blocks of ``block`` rows.  With bfloat16
    operands and blocks of 16 the product and the activation are one kernel."""
    _gpu(out, a, w_gate_up)
    M, I = out.shape
    if w_gate_up.shape[0] != 2 * I or a.shape != (M, w_gate_up.shape[1]) or out.dtype != a.dtype:
        raise KernelError(f"gemm_swiglu: shapes do not agree: a {tuple(a.shape)}, w {tuple(w_gate_up.shape)}, out {tuple(out.shape)}")
    if M == 0:
        return
    if _FAST and block == 16 and a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out.is_contiguous():
        from . import fast
        if fast.gemm_swiglu(out, a, w_gate_up, M, 2 * I, a.shape[1], _rows(a, "gemm a"), _rows(w_gate_up, "gemm w"), ws):
            return
    gu = torch.empty((M, 2 * I), dtype=a.dtype, device=a.device)
    gemm(gu, a, w_gate_up, ws=ws)
    swiglu(out, gu, block)


def gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, accumulate: bool = False,
         may_defer: bool = False, ws: Optional[KernelWorkspace] = None) -> None:
    """out[M, N] (+)= a[M, K] @ w[N, K]^T with float32 accumulation.

    ``ws``: where a product split over k keeps its pieces (without one, memory of this call's own).
    ``may_defer`` (with ``accumulate`` and ``ws``): the caller promises that ``out`` is next read
    by ``rmsnorm`` or ``materialize`` with the same workspace; a product that was split over k may
    then stay in pieces there."""
    if isinstance(a, KeyRanges):
        # attention's output of a decode step, its key ranges not merged yet: the weight-streaming
        # kernel merges them as it reads; anything else gets them merged first
        _gpu(out, w)
        if w.dim() != 2 or out.shape != (a.tokens, w.shape[0]) or w.shape[1] != a.heads * a.head_dim:
            raise KernelError(f"gemm: shapes do not agree: ranges [{a.tokens}, {a.heads} x {a.head_dim}], w {tuple(w.shape)}, out {tuple(out.shape)}")
        if accumulate:
            if out.dtype != torch.float32:
                raise KernelError("gemm: accumulation needs a float32 output")
            materialize(out, ws)
        from . import fast
        if _FAST and fast.gemm_from_ranges(out, a, w, accumulate, w.shape[0], _rows(w, "gemm w"), _rows(out, "gemm out"),
                                           may_defer and accumulate and out.is_contiguous(), ws):
            return
        merged = torch.empty((a.tokens, a.heads * a.head_dim), dtype=torch.bfloat16, device=out.device)
        fast.merge_ranges(merged, a)
        a = merged
    _gpu(out, a, w)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
        raise KernelError("gemm: operands must be 2-D")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N):
        raise KernelError(f"gemm: shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if accumulate and out.dtype != torch.float32:
        raise KernelError("gemm: accumulation needs a float32 output")
    lda, ldw, ldc = _rows(a, "gemm a"), _rows(w, "gemm w"), _rows(out, "gemm out")
    if M == 0:
        return
    if accumulate:
        materialize(out, ws)
    if _FAST and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        from . import fast
        if fast.gemm(out, a, w, accumulate, M, N, K, lda, ldw, ldc, may_defer and accumulate and out.is_contiguous(), ws):
            return
    _lib.call("core", "pi_gemm_general", out.data_ptr(), _dt(out), ldc, a.data_ptr(), _dt(a), lda, w.data_ptr(),
              _dt(w), ldw, M, N, K, int(accumulate), _stream())


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, hd: int, page_size: int, dtype) -> int:
    """Keys [pages, kv_heads, page, head_dim]; values transposed, [pages, kv_heads, head_dim, page]."""
    if (k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (nkv, page_size, hd)
            or tuple(v_cache.shape) != (k_cache.shape[0], nkv, hd, page_size)):
        raise KernelError(f"cache: expected keys [pages, {nkv}, {page_size}, {hd}] and values [pages, {nkv}, {hd}, {page_size}], "
                          f"got {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    if k_cache.dtype != dtype or v_cache.dtype != dtype or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise KernelError(f"cache: must be contiguous {dtype}, got {k_cache.dtype}")
    return k_cache.shape[0]


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """float32 [T, 2 * half]: cos then sin of float32(position) * inv_freq[j], for every token."""
    _gpu(positions, inv_freq)
    T, half = positions.shape[0], inv_freq.numel()
    _i32(positions, "positions")
    if inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous():
        raise KernelError("rope: the frequency table must be contiguous float32")
    table = torch.empty((T, 2 * half), dtype=torch.float32, device=positions.device)
    _lib.call("core", "pi_rope_table", table.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), T, half, _stream())
    return table


def _rotary_args(rotary, positions, T):
    """(table pointer, rotary_dim, interleaved) from ``rotary`` = (frequencies or table, R, interleaved)."""
    if rotary is None:
        return None, 0, False, None
    src, rdim, inter = rotary
    if src.dim() == 2:                       # already the step's cos / sin table
        if src.shape != (T, rdim) or src.dtype != torch.float32 or not src.is_contiguous():
            raise KernelError(f"rope: cos / sin table must be contiguous float32 [{T}, {rdim}]")
        return src.data_ptr(), rdim, inter, src
    if src.numel() != rdim // 2:
        raise KernelError(f"rope: frequency table must be float32 [{rdim // 2}]")
    table = rope_table(positions, src)
    return table.data_ptr(), rdim, inter, table


def qkv_projection(h: torch.Tensor, w_qkv: torch.Tensor, dtype: torch.dtype, ws: Optional[KernelWorkspace] = None):
    """h @ w_qkv^T for the attention mixer: a tensor [T, N] in ``dtype``, or - when the
    product was split over k and there is a workspace to keep them in - its pieces
    (``Partials``), which ``rope_kv_write`` sums on the fly so that the rotation sees float32
    values.  The pieces are good until the next product with the same workspace."""
    if _FAST and ws is not None and h.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and h.is_cuda:
        from . import fast
        p = fast.gemm_pieces(h, w_qkv, ws)
        if p is not None:
            ws.counts["qkv_pieces"] += 1
            return p
    out = torch.empty((h.shape[0], w_qkv.shape[0]), dtype=dtype, device=h.device)
    gemm(out, h, w_qkv, ws=ws)
    return out


def rope_kv_write(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], positions: torch.Tensor,
                  req_of_token: torch.Tensor, rotary, num_heads: int, num_kv_heads: int, head_dim: int,
                  k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  block_table: Optional[torch.Tensor], page_size: int, pieces=None, write_kv: Optional[bool] = None) -> None:
    """Rotate q in place by each token's position; rotate k and store k, v into the pages.

    ``rotary`` = (inv_freq float32 [R/2] or the step's cos / sin table [T, R], R, interleaved), or
    None for no rotation.
    ``k``/``v`` None: queries only (the layer reads a cache that another one writes).
    ``pieces``: the q|k|v projection still split over k (``fast.Partials`` with columns
    [q heads | k heads | v heads]); then ``q`` is the output buffer for the rotated queries and
    ``k``/``v`` are not given (``write_kv`` says whether the cache is written).
    """
    _gpu(q, k, v, positions, req_of_token, k_cache, v_cache, block_table)
    T = q.shape[0]
    check_attention_sizes(num_heads, num_kv_heads, head_dim)
    if q.shape[1] != num_heads * head_dim:
        raise KernelError(f"rope: q has {q.shape[1]} columns, expected {num_heads * head_dim}")
    _i32(positions, "positions", T)
    if pieces is not None:
        write = bool(write_kv)
        table_ptr, rdim, inter, _keep = _rotary_args(rotary, positions, T)
        q_size, kv_size = num_heads * head_dim, num_kv_heads * head_dim
        if pieces.M != T or pieces.N < q_size + (2 * kv_size if write else 0):
            raise KernelError(f"rope: pieces [{pieces.M}, {pieces.N}] do not hold q, k, v of {T} tokens")
        pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q.dtype) if write else 0
        _lib.call(
            "core", "pi_rope_kv_write", q.data_ptr(), _rows(q, "q"), None, 0, None, 0, _dt(q), positions.data_ptr(),
            _ptr(req_of_token) if write else None, table_ptr, rdim, int(bool(inter)), T, num_heads, num_kv_heads,
            head_dim, int(write), _ptr(k_cache) if write else None, _ptr(v_cache) if write else None,
            _ptr(block_table) if write else None, block_table.shape[1] if write else 0, page_size if write else 0, pages,
            pieces.part.data_ptr(), pieces.splits, pieces.N, 0, q_size, q_size + kv_size, _stream())
        return
    write = k is not None
    table_ptr, rdim, inter, _keep = _rotary_args(rotary, positions, T)
    if not write and rdim == 0:
        return
    pages = 0
    if write:
        if v is None or k.shape != (T, num_kv_heads * head_dim) or v.shape != k.shape or k.dtype != q.dtype or v.dtype != q.dtype:
            raise KernelError(f"rope: k/v must be [{T}, {num_kv_heads * head_dim}] of {q.dtype}")
        pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q.dtype)
        _i32(req_of_token, "req_of_token", T)
        if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
            raise KernelError("rope: block table must be contiguous int32 [requests, width]")
    _lib.call(
        "core", "pi_rope_kv_write", q.data_ptr(), _rows(q, "q"), _ptr(k), _rows(k, "k") if write else 0, _ptr(v),
        _rows(v, "v") if write else 0, _dt(q), positions.data_ptr(), _ptr(req_of_token) if write else None,
        table_ptr, rdim, int(bool(inter)), T, num_heads, num_kv_heads, head_dim, int(write),
        _ptr(k_cache) if write else None, _ptr(v_cache) if write else None, _ptr(block_table) if write else None,
        block_table.shape[1] if write else 0, page_size if write else 0, pages, None, 0, 0, 0, 0, 0, _stream())


def decode_attention_from_projection(out: torch.Tensor, qkv, ctx, rotary, num_heads: int, num_kv_heads: int,
                                     head_dim: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                     block_table: torch.Tensor, page_size: int, scale: float, window: int,
                                     write_kv: bool, ws: Optional[KernelWorkspace] = None, leave_ranges: int = 0):
    """For a step that holds single tokens only: rotation, cache write and attention in one
    kernel, from the q|k|v projection ``qkv`` (a tensor [T, N] or ``fast.Partials``, columns
    [q heads | k heads | v heads]).  Returns False, having done nothing, when the step, the
    sizes or the rotation (``rotary`` as for ``rope_kv_write``; only the whole head with paired
    halves, or none) are not what that kernel serves; the caller then takes the separate kernels.
    ``leave_ranges`` (needs ``ws``; 0, or the bytes of the weight matrix the result goes to): the
    caller hands the result straight to ``gemm`` with that matrix; when the keys were split into
    ranges, the kernel may then return them unmerged (``KeyRanges``, in the workspace) instead of
    filling ``out``, and the product merges them as it reads."""
    if not (_FAST and out.dtype == torch.bfloat16 and out.is_cuda and getattr(ctx, "all_decode", False)):
        return False
    from . import fast
    if not isinstance(qkv, Partials) and qkv.dtype != torch.bfloat16:
        return False
    T = out.shape[0]
    table = None
    if rotary is not None:
        src, rdim, inter = rotary
        if rdim != head_dim or inter:
            return False
        _ptr_unused, _rdim, _inter, table = _rotary_args(rotary, ctx.positions, T)
    check_attention_sizes(num_heads, num_kv_heads, head_dim)
    if out.shape != (T, num_heads * head_dim):
        raise KernelError(f"attention: out {tuple(out.shape)} does not match {num_heads} x {head_dim}")
    pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, out.dtype)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
        raise KernelError("attention: block table must be contiguous int32 [requests, width]")
    return fast.decode_attention_from_projection(out, qkv, ctx, table, num_heads, num_kv_heads, head_dim, k_cache, v_cache,
                                                 block_table, page_size, scale, window, pages, write_kv, ws, leave_ranges)


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, ctx, num_heads: int, num_kv_heads: int, head_dim: int,
                    page_size: int, scale: float, window: int = 0, ws: Optional[KernelWorkspace] = None) -> None:
    """Causal attention of every token of the step over its request's pages.

    ``ctx`` carries ``positions`` and ``req_of_token`` ([T] int32), the step's shape on the host
    (``q_lens``, ``kv_lens``, ``all_decode``) and, in ``plans``, the work lists that the
    matrix-core kernels want (made here when the step function has not).
    """
    _gpu(out, q, k_cache, v_cache, block_table, ctx.positions, ctx.req_of_token)
    T = q.shape[0]
    check_attention_sizes(num_heads, num_kv_heads, head_dim)
    if q.shape[1] != num_heads * head_dim or out.shape != (T, num_heads * head_dim) or out.dtype != q.dtype:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not match {num_heads} x {head_dim}")
    pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q.dtype)
    _i32(ctx.positions, "positions", T)
    _i32(ctx.req_of_token, "req_of_token", T)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
        raise KernelError("attention: block table must be contiguous int32 [requests, width]")
    if T == 0:
        return
    if _FAST and q.dtype == torch.bfloat16:
        from . import fast
        if fast.paged_attention(out, q, k_cache, v_cache, block_table, ctx, num_heads, num_kv_heads, head_dim,
                                page_size, scale, window, pages, ws):
            return
    # a step of few tokens over long contexts: its keys cut into ranges, merged by a second kernel
    # (as many as the context-length bucket asks for, so that a step gives the same bits eagerly and replayed)
    ranges = general_attention_ranges(T, num_heads, int(ctx.max_kv_len))
    part = torch.empty(T * num_heads * ranges * (head_dim + 2), dtype=torch.float32, device=q.device) if ranges > 1 else None
    _lib.call("core", "pi_paged_attention_general", out.data_ptr(), _rows(out, "attention out"), q.data_ptr(),
              _rows(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), _dt(q), block_table.data_ptr(),
              block_table.shape[1], ctx.req_of_token.data_ptr(), ctx.positions.data_ptr(), T, num_heads,
              num_kv_heads, head_dim, page_size, float(scale), int(window), pages, ranges, _ptr(part),
              0 if part is None else part.numel(), _stream())


def general_attention_ranges(tokens: int, num_heads: int, max_kv_len: int) -> int:
    """Key ranges per (token, head) that the general attention kernel makes for such a step."""
    return int(_lib.load("core").pi_paged_attention_general_ranges(tokens, num_heads, decode_length_bucket(max_kv_len)))


def sample(out: torch.Tensor, logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None, ws: Optional[KernelWorkspace] = None) -> None:
    """out[m] = argmax of row m (lowest index among equals) where temperature[m] <= 0 or
    no temperatures are given; otherwise the first index whose cumulative
    softmax(logits / temperature) reaches uniform[m]."""
    _gpu(out, logits, temperature, uniform)
    M, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    _i32(out, "sample out", M)
    for t, what in ((temperature, "temperature"), (uniform, "uniform")):
        if t is not None and (t.dtype != torch.float32 or t.numel() < M or not t.is_contiguous()):
            raise KernelError(f"sample: {what} must be contiguous float32 [{M}]")
    if temperature is not None and uniform is None:
        raise KernelError("sample: temperatures given without uniform numbers")
    chunks = _lib.load("core").pi_sample_chunks(V)
    if chunks == 0:
        part = None
    elif ws is not None:
        part = ws.sample_part
    else:
        part = torch.empty(M * chunks * 4, dtype=torch.float32, device=logits.device)
    _lib.call("core", "pi_sample", out.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), _ptr(temperature),
              _ptr(uniform), M, V, _ptr(part), 0 if part is None else part.numel(), _stream())


# ----------------------------------------------------------------------------- work lists
def decode_length_bucket(max_kv_len: int) -> int:
    """The context-length bucket that decides a decode step's attention key ranges."""
    from . import fast
    return fast.decode_length_bucket(max_kv_len)


def attention_planner(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                      window: int, device):
    """What makes a step's work lists for an attention mixer of these sizes (a hashable object with
    ``plan(q_lens, kv_lens)``; equal ones share a plan), or None when its kernels need none."""
    if _FAST and dtype == torch.bfloat16 and _lib.build.MODULES["bf16"]:
        from . import fast
        return fast.attention_planner(dtype, num_heads, num_kv_heads, head_dim, page_size, int(window), torch.device(device))
    return None


def upload_arrays(arrays, device):
    """int32 host arrays by name -> device views of one packed copy."""
    from . import fast
    return fast.upload_arrays(arrays, device)
