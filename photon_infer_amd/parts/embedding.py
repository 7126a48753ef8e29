"""Token embedding and output head.

Embedding is a row gather without scaling (src/ops/kernels/cuda/embedding_kernel.cu:31-63);
the head is ``logits = h W^T`` in float32 without bias or scaling
(src/arch/llama_model.cpp:256,601).  A tied head uses the embedding's tensor itself
(the reference copies it, src/io/checkpoint.cpp:305-313).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import Part


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec("weight", (self.vocab_size, self.hidden_size), "table")]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.weight = tensors["weight"]

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """int32 [T] -> float32 residual stream [T, hidden]."""
        x = torch.empty((token_ids.shape[0], self.hidden_size), dtype=torch.float32, device=token_ids.device)
        ops.embedding(x, self.weight, token_ids)
        return x


class LMHead(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.tied = bool(tied)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [] if self.tied else [TensorSpec("weight", (self.vocab_size, self.hidden_size))]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device, tied_weight: Optional[torch.Tensor] = None) -> None:
        super().load(tensors, dtype, device)
        self.weight = tied_weight if self.tied else tensors["weight"]

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.weight]

    def forward(self, h: torch.Tensor, ctx=None) -> torch.Tensor:
        """activations [M, hidden] -> float32 logits [M, vocab]."""
        logits = torch.empty((h.shape[0], self.vocab_size), dtype=torch.float32, device=h.device)
        ops.gemm(logits, h, self.weight, ws=ctx.workspace if ctx is not None else None)
        return logits
