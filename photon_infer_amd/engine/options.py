"""Engine options: every constant the reference scatters through its sources
(chunk 256 and max_sequences 32 in include/photon/scheduler/continuous_batch_engine.hpp:61-66,
block size 16 and the pool size in demo/batched_infer_multi_prompts.cpp:355-358) as a field.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..errors import PhotonError

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float32):
            return name
        raise PhotonError(f"compute dtype must be bfloat16 or float32, got {name}")
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise PhotonError(f"compute dtype must be bfloat16 or float32, got '{name}'") from None


@dataclass
class EngineOptions:
    dtype: object = "bfloat16"           # compute dtype: "bfloat16" or "float32"
    block_size: int = 16                 # tokens per cache page
    num_blocks: Optional[int] = None     # pages per cache group; None: from max_cache_tokens
    max_cache_tokens: Optional[int] = None  # tokens the page pool holds; None: max_batch * max_model_len, or as many
                                         # as fit into memory_fraction of the device memory that is free after the weights
    memory_fraction: float = 0.9         # share of the free device memory that a pool sized by default may take
    max_batch: int = 32                  # most live requests (= state slots)
    max_step_tokens: int = 2048          # token budget of one step
    chunk_size: int = 512                # largest prompt portion of one request in one step (the reference: 256; here a
                                         # step of 512 tokens costs little more than one of 256)
    max_model_len: Optional[int] = None  # longest sequence; None: the model's max positions
    seed: int = 0
    device: str = "cuda:0"
    stream_copies: Optional[bool] = None  # bfloat16 only: keep a second copy of the weight matrices in the order the
                                         # weight-streaming kernels read them (steps of up to 128 tokens are 2 to 4 % faster;
                                         # costs the matrices' size in device memory again).  None: if they take at most half
                                         # of the memory that is free after the weights; True: always, or an error; False: never.
                                         # The copies are made at load: weights must not be changed afterwards.
    use_graphs: bool = True              # replay HIP graphs for decode-only steps
    keep_logits: bool = False            # keep a decode step's float32 logits readable until the next decode step
                                         # (ModelRunner.decode_logits, [requests, vocab]); costs that much memory per graph
    lookahead: bool = True               # schedule a decode step while the one before it still runs (needs use_graphs)

    def resolved_dtype(self) -> torch.dtype:
        return parse_dtype(self.dtype)
