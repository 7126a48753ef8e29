"""Causal grouped-query attention over the paged cache.

Formulas (include/photon/ops/kernels/mha_kernel.hpp:174-230): for a query at absolute
position p, head n, kv head ``g = n // (heads / kv_heads)``:
``s_t = scale * <q_n, K_g[t]>`` for t = 0..p (causality is the loop bound),
``P = softmax(s)``, ``o_n = sum_t P_t V_g[t]``; heads are concatenated and projected by
``o_proj``.  Projections have no bias and weights are ``[out, in]`` with ``y = x W^T``
(src/arch/transformer_block.cpp:204-211,262-270).  Keys are stored after the position
encoding, values as they are (src/ops/kernels/cuda/paged_kv_write.cu:27-77).

Unlike the reference's batched path (src/arch/transformer_block.cpp:443-509), every
token carries its own position and sees only keys at positions <= its own, so a
prompt may be cut into portions anywhere.

An optional ``window`` W restricts a query at p to keys p-W+1..p.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import MIXERS, KVCacheSpec, LayerCache, Mixer, PositionEncoding, StepContext


POSITION_PREFIX = "position."


class PagedAttention(Mixer):
    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: Optional[PositionEncoding] = None,
        scale: Optional[float] = None,
        window: Optional[int] = None,
        own_kv: bool = True,
    ):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.position = position
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.window = int(window) if window else None
        self.own_kv = bool(own_kv)  # False: the layer has no k/v projection and reads another's cache
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        ops.check_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec("q_proj.weight", (self.q_size, self.hidden_size))]
        if self.own_kv:
            specs += [
                TensorSpec("k_proj.weight", (self.kv_size, self.hidden_size)),
                TensorSpec("v_proj.weight", (self.kv_size, self.hidden_size)),
            ]
        specs.append(TensorSpec("o_proj.weight", (self.hidden_size, self.q_size)))
        if self.position is not None:     # a position encoding with tensors of its own keeps them under "position."
            specs += [s.with_prefix(POSITION_PREFIX) for s in self.position.tensor_specs()]
        return specs

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    @property
    def graph_safe(self) -> bool:
        # the kernels take the step's shape from device memory; a position encoding applied by
        # library calls must make the promise itself
        return self.position is None or bool(self.position.graph_safe)

    def step_planner(self, page_size: int):
        return ops.attention_planner(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim, page_size,
                                     self.window or 0, self.device)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        mats = [tensors["q_proj.weight"]]
        if self.own_kv:
            mats += [tensors["k_proj.weight"], tensors["v_proj.weight"]]
        # one projection for q, k and v: rows [q heads | k heads | v heads]
        common = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = torch.cat([m.to(common) for m in mats], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        if self.position is not None:
            own = {n[len(POSITION_PREFIX):]: t for n, t in tensors.items() if n.startswith(POSITION_PREFIX)}
            self.position.load(own, dtype, device)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_qkv, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T = h.shape[0]
        writes = self.own_kv and cache.writes
        rotary = self.position.rotary_params(ctx) if self.position is not None else None
        fused_position = self.position is None or rotary is not None
        table = ctx.block_tables[cache.group]
        ws = ctx.workspace
        qkv = ops.qkv_projection(h, self.w_qkv, self.dtype, ws) if fused_position else None
        if qkv is not None and ctx.all_decode:
            # single tokens only: one kernel rotates, writes the cache and attends
            attn = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
            done = ops.decode_attention_from_projection(attn, qkv, ctx, rotary, self.num_heads, self.num_kv_heads,
                                                        self.head_dim, cache.k, cache.v, table, cache.page_size, self.scale,
                                                        self.window or 0, writes, ws,
                                                        leave_ranges=self.w_o.numel() * self.w_o.element_size())
            if done:
                # the output, or its key ranges still to be merged, which the product does as it reads them
                ops.gemm(x, done if isinstance(done, ops.KeyRanges) else attn, self.w_o, accumulate=True, may_defer=getattr(ctx, "may_defer", False), ws=ws)
                return
        if qkv is not None and not isinstance(qkv, torch.Tensor):
            # the projection is still in pieces (split over k): the rotation kernel sums them
            q = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
            ops.rope_kv_write(q, None, None, ctx.positions, ctx.req_of_token, rotary, self.num_heads,
                              self.num_kv_heads, self.head_dim, cache.k, cache.v, table, cache.page_size,
                              pieces=qkv, write_kv=writes)
        else:
            if qkv is None:
                qkv = torch.empty((T, self.w_qkv.shape[0]), dtype=self.dtype, device=h.device)
                ops.gemm(qkv, h, self.w_qkv, ws=ws)
            q = qkv[:, : self.q_size]
            k = qkv[:, self.q_size : self.q_size + self.kv_size] if self.own_kv else None
            v = qkv[:, self.q_size + self.kv_size :] if self.own_kv else None
            if not fused_position:
                self.position.apply(q, k, ctx)
            ops.rope_kv_write(
                q, k if writes else None, v if writes else None, ctx.positions, ctx.req_of_token,
                rotary, self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v, table, cache.page_size,
            )
        attn = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
        ops.paged_attention(
            attn, q, cache.k, cache.v, table, ctx,
            self.num_heads, self.num_kv_heads, self.head_dim, cache.page_size,
            self.scale, self.window or 0, ws,
        )
        # where the arrangement allows it, the product stays in pieces for the stream's next reader
        ops.gemm(x, attn, self.w_o, accumulate=True, may_defer=getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("attention", PagedAttention)
