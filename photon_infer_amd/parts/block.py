"""Arrangements of norm, mixer and feed-forward around the residual stream.

Pre-norm order of the reference (include/photon/arch/transformer_block.hpp:34-51,
src/arch/transformer_block.cpp:189-299):
``x += mixer(norm1(x)); x += ffn(norm2(x))``.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import BLOCKS, Block, FeedForward, LayerCache, Mixer, Norm, Part, StepContext


class PreNormBlock(Block):
    """Each of the four parts comes with the name prefix of its tensors inside the block."""

    def __init__(self, norm1: Tuple[str, Norm], mixer: Tuple[str, Mixer],
                 norm2: Tuple[str, Norm], ffn: Tuple[str, FeedForward]):
        self._named: List[Tuple[str, Part]] = [norm1, mixer, norm2, ffn]
        self.norm1, self.mixer, self.norm2, self.ffn = norm1[1], mixer[1], norm2[1], ffn[1]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s.with_prefix(p) for p, part in self._named for s in part.tensor_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        for prefix, part in self._named:
            part.load({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._named)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for _, part in self._named for w in part.streamed_weights()]

    @property
    def reads_deferred(self) -> bool:
        return bool(getattr(self.norm1, "consumes_deferred", False))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        # A mixer or feed-forward may leave its update of x in pieces (ops.gemm(..., may_defer=True))
        # when the stream's next reader adds them: norm2 after the mixer; after the feed-forward,
        # whoever the model says reads the stream next.
        ctx.may_defer = bool(getattr(self.norm2, "consumes_deferred", False))
        self.mixer.forward(self.norm1.forward(x, ctx), x, ctx, cache)
        ctx.may_defer = ctx.after_block_consumes
        self.ffn.forward(self.norm2.forward(x, ctx), x, ctx)
        ctx.may_defer = False


BLOCKS.register("prenorm", PreNormBlock)
