"""A decoder model as data: embedding, a list of blocks, a run order, final norm, head.

Reference: src/arch/llama_model.cpp:30-46 builds embedding + N identical blocks +
final norm + classifier and runs them in index order (:242-246, :583-593).  Here the
run order is a list of entries; an entry names the block whose weights it runs and,
optionally, an earlier entry whose cache it reads instead of writing one of its own.
A block may appear in several entries.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..errors import ConfigError
from ..weights.loader import TensorSpec
from .base import Block, KVCacheSpec, LayerCache, Norm, PagedCacheSpec, PagedTensor, StateSpec, StepContext
from .embedding import LMHead, TokenEmbedding


@dataclass(frozen=True)
class RunEntry:
    layer: int                       # index into ModelSpec.layers
    cache_of: Optional[int] = None   # index of an earlier RunEntry whose cache is read


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: Tuple[str, TokenEmbedding]
    layers: List[Tuple[str, Block]]
    final_norm: Tuple[str, Norm]
    head: Tuple[str, LMHead]
    run_order: List[RunEntry] = field(default_factory=list)
    ignorable: Tuple[str, ...] = ()   # name patterns a folder may hold beyond the expected ones
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    def __post_init__(self):
        if not self.run_order:
            self.run_order = [RunEntry(i) for i in range(len(self.layers))]
        for i, e in enumerate(self.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ConfigError(f"run order entry {i} names layer {e.layer} of {len(self.layers)}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ConfigError(f"run order entry {i} reads the cache of entry {e.cache_of}, which is not earlier")
                if self.run_order[e.cache_of].cache_of is not None:
                    raise ConfigError(f"run order entry {i} reads the cache of entry {e.cache_of}, which owns none")

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s.with_prefix(self.embedding[0]) for s in self.embedding[1].tensor_specs()]
        for prefix, block in self.layers:
            specs += [s.with_prefix(prefix) for s in block.tensor_specs()]
        specs += [s.with_prefix(self.final_norm[0]) for s in self.final_norm[1].tensor_specs()]
        specs += [s.with_prefix(self.head[0]) for s in self.head[1].tensor_specs()]
        return specs


# ------------------------------------------------------------------ what the cache must hold
# A cache or a state belongs to one mixer of one run-order entry: the key (entry index, index of
# the mixer among the block's ``mixers()``).
CacheKey = Tuple[int, int]


@dataclass(frozen=True)
class CacheGroupPlan:
    """Mixers whose paged tensors follow one block table (the same window)."""

    window: Optional[int]
    owners: Tuple[CacheKey, ...]                        # the mixers that own pages
    tensors: Tuple[Tuple[PagedTensor, ...], ...]        # per owner: what it keeps per token


@dataclass(frozen=True)
class CachePlan:
    groups: Tuple[CacheGroupPlan, ...]
    states: Tuple[Tuple[CacheKey, StateSpec], ...]
    group_of: Dict[CacheKey, int]                       # also for mixers that read another entry's pages
    owner_of: Dict[CacheKey, CacheKey]                  # whose cache or state a mixer uses (itself, or its ``cache_of`` entry's)


def plan_cache(spec: ModelSpec) -> CachePlan:
    """Group the run order's cache needs: one block table per distinct window."""
    by_window: Dict[Optional[int], List[Tuple[CacheKey, tuple]]] = {}
    states: List[Tuple[CacheKey, StateSpec]] = []
    owner_of: Dict[CacheKey, CacheKey] = {}
    for i, e in enumerate(spec.run_order):
        for j, mixer in enumerate(spec.layers[e.layer][1].mixers()):
            if e.cache_of is not None:
                owner_of[(i, j)] = (e.cache_of, j)
                continue
            owner_of[(i, j)] = (i, j)
            if not getattr(mixer, "own_kv", True):
                raise ConfigError(f"run order entry {i}: layer {e.layer} writes no keys or values of its own and "
                                  f"must name the entry whose cache it reads")
            need = mixer.cache_spec()
            if isinstance(need, (KVCacheSpec, PagedCacheSpec)):
                by_window.setdefault(need.window, []).append(((i, j), tuple(need.tensors)))
            elif isinstance(need, StateSpec):
                states.append(((i, j), need))
            elif need is not None:
                raise ConfigError(f"mixer {j} of layer {e.layer} returned an unknown cache spec {need!r}")
    groups, group_of = [], {}
    for g, (window, items) in enumerate(sorted(by_window.items(), key=lambda kv: (kv[0] is not None, kv[0] or 0))):
        groups.append(CacheGroupPlan(window, tuple(k for k, _ in items), tuple(t for _, t in items)))
        for k, _ in items:
            group_of[k] = g
    for key, owner in owner_of.items():
        if owner in group_of:
            group_of[key] = group_of[owner]
    return CachePlan(tuple(groups), tuple(states), group_of, owner_of)


# ------------------------------------------------------------------ the runnable model
class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = spec.embedding[1]
        self.blocks = [b for _, b in spec.layers]
        self.final_norm = spec.final_norm[1]
        self.head = spec.head[1]
        self.dtype: Optional[torch.dtype] = None

    def load(self, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device) -> None:
        """Hand each part its tensors (names relative to the part's prefix)."""
        device = torch.device(device)
        self.dtype, self.device = dtype, device

        def sub(prefix: str) -> Dict[str, torch.Tensor]:
            return {n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}

        self.embedding.load(sub(self.spec.embedding[0]), dtype, device)
        for prefix, block in self.spec.layers:
            block.load(sub(prefix), dtype, device)
        self.final_norm.load(sub(self.spec.final_norm[0]), dtype, device)
        # a head that is tied takes the embedding's matrix itself
        self.head.load(sub(self.spec.head[0]), dtype, device, tied_weight=getattr(self.embedding, "weight", None))

    def forward(self, ctx: StepContext, caches: Sequence) -> Optional[torch.Tensor]:
        """Run the step's tokens through the run order; float32 logits [M, vocab] at
        ``ctx.logit_rows`` (None when no row is wanted).  ``caches``: per run-order entry its
        ``LayerCache`` (a list of them for a block of several mixers)."""
        ws = ctx.workspace
        ops.reset_deferred(ws)             # nothing of an earlier (failed) step may linger
        ctx.scratch.clear()
        x = self.embedding.forward(ctx.token_ids)
        order = self.spec.run_order
        wanted = ctx.logit_rows.shape[0] > 0
        for i, entry in enumerate(order):
            block = self.blocks[entry.layer]
            # A block meets an update of the stream that is still in pieces only if it says that
            # its first reader adds them, and may leave one behind only for such a reader.
            if not block.reads_deferred:
                ops.materialize(x, ws)
            if i + 1 < len(order):
                ctx.after_block_consumes = bool(self.blocks[order[i + 1].layer].reads_deferred)
            else:                          # the final norm; or nobody (the pieces are then dropped unread)
                ctx.after_block_consumes = not wanted or bool(getattr(self.final_norm, "consumes_deferred", False))
            ctx.may_defer = False
            block.forward(x, ctx, caches[i])
        ctx.may_defer = ctx.after_block_consumes = False
        if not wanted:
            ops.discard_deferred(x, ws)    # the stream is not read again
            return None
        if not getattr(self.final_norm, "consumes_deferred", False):
            ops.materialize(x, ws)
        return self.head.forward(self.final_norm.forward(x, ctx, rows=ctx.logit_rows), ctx)

    def streamed_weights(self) -> List[torch.Tensor]:
        """The weight matrices that every decode step reads whole (see ``Part.streamed_weights``)."""
        parts = [self.embedding, self.final_norm, self.head] + self.blocks
        return [w for p in parts for w in getattr(p, "streamed_weights", lambda: [])()]

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be captured as a HIP graph: every part of the
        run order, the embedding, the final norm and the head promise it."""
        parts = [self.embedding, self.final_norm, self.head] + [self.blocks[e.layer] for e in self.spec.run_order]
        return all(getattr(p, "graph_safe", False) for p in parts)
