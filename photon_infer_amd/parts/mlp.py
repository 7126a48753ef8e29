"""Gated feed-forward (SwiGLU).

Formula (src/arch/transformer_block.cpp:282-295, include/photon/ops/kernels/swiglu_kernel.hpp:52-76):
``g = h W1^T``, ``u = h W3^T``, ``a = g / (1 + exp(-g)) * u``, ``x += a W2^T``; no bias.
Tensor names: ``gate_proj`` = W1, ``up_proj`` = W3, ``down_proj`` = W2.  The sigmoid
and the product run in float32.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import FEED_FORWARDS, FeedForward, StepContext

INTERLEAVE = 16   # rows of a matrix-core tile


class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation != "silu":
            raise UnsupportedModelError(f"gated feed-forward activation '{activation}' is not supported")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)

    def tensor_specs(self) -> List[TensorSpec]:
        I, D = self.intermediate_size, self.hidden_size
        return [
            TensorSpec("gate_proj.weight", (I, D)),
            TensorSpec("up_proj.weight", (I, D)),
            TensorSpec("down_proj.weight", (D, I)),
        ]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        common = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        g, u = g.to(common), u.to(common)
        I = self.intermediate_size
        if common == torch.bfloat16 and I % INTERLEAVE == 0:
            # one projection for gate and up, rows interleaved in blocks of 16 (gate block, up
            # block, ...): the matrix-core kernels then hold a feature's gate and up value in
            # the same lane and apply the activation before anything is stored
            self.interleave = INTERLEAVE
            self.w_gate_up = torch.stack([g.view(I // INTERLEAVE, INTERLEAVE, -1), u.view(I // INTERLEAVE, INTERLEAVE, -1)],
                                         dim=1).reshape(2 * I, -1).contiguous()
        else:
            self.interleave = 0                      # rows [gate | up]
            self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_gate_up, self.w_down]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        act = torch.empty((h.shape[0], self.intermediate_size), dtype=self.dtype, device=h.device)
        ws = ctx.workspace if ctx is not None else None
        ops.gemm_swiglu(act, h, self.w_gate_up, self.interleave, ws=ws)
        ops.gemm(x, act, self.w_down, accumulate=True, may_defer=getattr(ctx, "may_defer", False), ws=ws)


FEED_FORWARDS.register("swiglu", SwiGLU)
