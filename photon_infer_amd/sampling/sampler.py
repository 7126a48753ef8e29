"""Choosing the next token: greedy and temperature sampling, on the GPU.

Reference: greedy = arg max with the first maximum winning (src/arch/llama_model.cpp:304-328,
GPU: src/ops/kernels/cuda/sampling_kernel.cu); temperature = softmax((l - max) / T) and the
first index whose cumulative probability reaches a uniform draw (demo/llama_infer.cpp:77-101,
T = 0.8 and ``rand()`` there).  The reference accepts ``top_p`` in its web server and
ignores it (web/web_server.cpp:147,449); nothing else is sampled with.

The uniform draw is a pure function of (seed, draw index), so what a request samples
does not depend on which other requests share its batch or on whether it was preempted
and recomputed.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_draw(seed: int, index: int) -> float:
    """Draw number ``index`` of the stream ``seed``: a float32-exact value in (0, 1)."""
    h = _splitmix64(_splitmix64(seed & _MASK) ^ ((index * 0xD6E8FEB86659FD93) & _MASK))
    return ((h >> 40) + 0.5) / float(1 << 24)


@dataclass
class SamplingParams:
    temperature: float = 0.0          # 0 = greedy
    max_new_tokens: int = 128
    seed: int = 0
    ignore_eos: bool = False


class Sampler:
    def __init__(self, device, workspace=None):
        """``workspace``: the runner's ``ops.KernelWorkspace`` (scratch of the sampling kernels)."""
        self.device = torch.device(device)
        self.workspace = workspace

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        """One token per row of float32 ``logits`` [M, V]."""
        M = logits.shape[0]
        out = torch.empty(M, dtype=torch.int32, device=logits.device)
        if any(t > 0 for t in temperatures):
            host = np.asarray([list(temperatures), list(uniforms)], np.float32)
            dev = torch.from_numpy(host).to(logits.device)
            ops.sample(out, logits, dev[0], dev[1], ws=self.workspace)
        else:
            ops.sample(out, logits, ws=self.workspace)
        return out.cpu().tolist()

    def greedy(self, logits: torch.Tensor) -> List[int]:
        return self.sample(logits, [0.0] * logits.shape[0], [0.0] * logits.shape[0])
