"""Rotary position encoding with optional frequency scaling.

Reference formula (include/photon/ops/kernels/rope_kernel.hpp:55-84,126-165): pair j of
a head is rotated by ``angle = pos * f_j`` with ``f_j = base^(-2j/head_size)``:
``(a, b) <- (a cos - b sin, a sin + b cos)``.  The reference fixes base = 10000, pairs
neighbours ``(x[2j], x[2j+1])`` and tabulates sin/cos per position; here the base, the
scaling rule, the pairing and the rotated width are parameters, and only the
frequencies are tabulated (built in float64, kept in float32); the angle and its
sine / cosine are computed in float32 inside the kernel from the token's position.

llama3 scaling (not in the reference): with wavelength ``lam = 2*pi / f``,
``L`` = original context, ``lo``/``hi`` = low/high frequency factors:
``lam < L/hi`` keeps f; ``lam > L/lo`` gives f/factor; between them
``s = (L/lam - lo) / (hi - lo)`` and ``f <- (1 - s) * f/factor + s * f``.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..errors import UnsupportedModelError
from .base import POSITION_ENCODINGS, PositionEncoding


def rope_frequencies(rotary_dim: int, theta: float, scaling=None) -> torch.Tensor:
    """float64 tensor [rotary_dim / 2] of per-pair frequencies."""
    half = rotary_dim // 2
    j = torch.arange(half, dtype=torch.float64)
    freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * j / rotary_dim)
    if scaling is None:
        return freq
    if scaling.rope_type == "linear":
        return freq / scaling.factor
    if scaling.rope_type == "llama3":
        L = float(scaling.original_max_position_embeddings)
        lo, hi, factor = scaling.low_freq_factor, scaling.high_freq_factor, scaling.factor
        wavelen = 2.0 * math.pi / freq
        smooth = (L / wavelen - lo) / (hi - lo)
        mid = (1.0 - smooth) * freq / factor + smooth * freq
        out = torch.where(wavelen > L / lo, freq / factor, freq)
        is_mid = (wavelen <= L / lo) & (wavelen >= L / hi)
        return torch.where(is_mid, mid, out)
    raise UnsupportedModelError(f"rope scaling '{scaling.rope_type}' is not supported")


class RotaryEmbedding(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int, theta: float, scaling=None, interleaved: bool = False,
                 rotary_dim: Optional[int] = None):
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise UnsupportedModelError(
                f"rotary_dim must be even and within head_dim, got {self.rotary_dim} / {self.head_dim}"
            )
        self.theta = float(theta)
        self.scaling = scaling
        self.interleaved = bool(interleaved)
        self.inv_freq: Optional[torch.Tensor] = None

    def load(self, tensors, dtype, device) -> None:
        super().load(tensors, dtype, device)
        if self.inv_freq is None or self.inv_freq.device != device:
            self.inv_freq = rope_frequencies(self.rotary_dim, self.theta, self.scaling).to(
                dtype=torch.float32, device=device
            )

    def rotary_params(self, ctx=None):
        """(frequencies, rotated width, pairing) - or, given the step's context, the step's
        cos / sin table instead of the frequencies: every layer of a step rotates by the same
        angles, so they are computed once."""
        if ctx is None:
            return self.inv_freq, self.rotary_dim, self.interleaved
        table = ctx.scratch.get(("rope", id(self)))
        if table is None:
            from .. import ops
            table = ctx.scratch[("rope", id(self))] = ops.rope_table(ctx.positions, self.inv_freq)
        return table, self.rotary_dim, self.interleaved


POSITION_ENCODINGS.register("rope", RotaryEmbedding)
