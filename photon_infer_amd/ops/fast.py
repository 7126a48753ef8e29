"""Dispatch to the bfloat16 matrix-core kernels (module "bf16").

Each function returns True when it ran the operation and False when the sizes are not
ones its kernels take, in which case the caller uses the general kernel.
"""
from __future__ import annotations


def gemm(out, a, w, accumulate, M, N, K, lda, ldw, ldc) -> bool:
    return False


def paged_attention(out, q, k_cache, v_cache, block_table, ctx, num_heads, num_kv_heads, head_dim,
                    page_size, scale, window, pages) -> bool:
    return False


def plan_attention(q_lens, kv_lens) -> dict:
    return {}


def attach_attention_plan(ctx, plan, views) -> None:
    pass
