"""RMS normalisation part.

Formula (include/photon/ops/kernels/rmsnorm_kernel.hpp:55-87): mean of squares over
the row, ``rms = sqrt(mean + eps)`` with eps inside the root, ``y = w * (x / rms)``;
no mean-centring, no bias.  Sum, root and scaling run in float32; the result is
rounded once to the compute dtype.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import NORMS, Norm


class RMSNorm(Norm):
    consumes_deferred = True   # reads the stream through ops.rmsnorm, which adds a pending update
    graph_safe = True

    def __init__(self, dim: int, eps: float):
        self.dim = int(dim)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec("weight", (self.dim,), "norm")]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor, ctx=None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        m = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((m, self.dim), dtype=self.dtype, device=x.device)
        ops.rmsnorm(out, x, self.weight, self.eps, rows, ws=ctx.workspace if ctx is not None else None)
        return out


NORMS.register("rmsnorm", RMSNorm)
