"""Per-request state of fixed size, indexed by the request's slot.

The reference has nothing of this kind (its nearest relative is the per-batch buffer
``sampled_tokens_gpu_``, include/photon/scheduler/continuous_batch_engine.hpp:70).  A mixer
that keeps a recurrent state declares its shape; the engine keeps one slab
``[max_slots, *shape]`` per such run-order entry and clears a slot's row when a request
is admitted to it.  An architecture without such mixers has no slabs.
"""
from __future__ import annotations

from typing import Dict, Sequence, Tuple

import torch


class StateSlots:
    def __init__(self, specs: Sequence[Tuple[int, object]], max_slots: int, device):
        """``specs``: (key, StateSpec) pairs; a key names the mixer that owns the state (run-order entry, mixer index)."""
        self.max_slots = int(max_slots)
        self.slabs: Dict[object, torch.Tensor] = {
            entry: torch.zeros((self.max_slots, *spec.shape), dtype=spec.dtype, device=device)
            for entry, spec in specs
        }

    def get(self, entry):
        return self.slabs.get(entry)

    def clear(self, slot: int) -> None:
        for slab in self.slabs.values():
            slab[slot].zero_()

    @property
    def bytes_per_slot(self) -> int:
        return sum(s[0].numel() * s.element_size() for s in self.slabs.values())
