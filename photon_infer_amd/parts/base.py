"""Interfaces of the parts a layer is put together from, and their registries.

A model is data: a list of blocks, each naming a norm, a mixer, a feed-forward and an
arrangement, plus a run order.  Every part takes its sizes and constants as
constructor parameters, declares the tensors it expects (relative names) and what it
needs from the cache manager; none of them knows which model it sits in.

The reference wires one fixed block (src/arch/transformer_block.cpp:28-58: two norms,
seven matmuls, rope, mha, add, swiglu) and has no such seam; the interfaces below are
what replaces it.

Data flow convention: the residual stream ``x`` is float32 ``[T, hidden]`` in both
compute modes.  A norm reads ``x`` and writes activations ``h`` in the compute dtype;
a mixer or feed-forward reads ``h`` and *adds* its result into ``x``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec


# --------------------------------------------------------------------------- cache needs
PAGE = -1     # in a paged tensor's shape: the axis that holds a page's tokens


@dataclass(frozen=True)
class PagedTensor:
    """One tensor that a mixer keeps per token, in pages: the shape of one page of it, with ``PAGE``
    standing for the page's tokens, e.g. keys ``(kv_heads, PAGE, head_dim)``, values transposed
    ``(kv_heads, head_dim, PAGE)``, one latent vector per token ``(PAGE, width)``.  The pool is
    ``[pages, *shape]``.  ``dtype`` None: the compute dtype."""

    name: str
    shape: tuple
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> tuple:
        if sum(1 for d in self.shape if d == PAGE) != 1:
            raise UnsupportedModelError(f"paged tensor '{self.name}': its shape {self.shape} must name the page axis once")
        return tuple(page_size if d == PAGE else int(d) for d in self.shape)

    def page_bytes(self, page_size: int, compute_dtype: torch.dtype) -> int:
        n = 1
        for d in self.page_shape(page_size):
            n *= d
        return n * torch.empty((), dtype=self.dtype or compute_dtype).element_size()


@dataclass(frozen=True)
class PagedCacheSpec:
    """What a mixer keeps per token, in pages: any number of named tensors, each with its own
    shape and layout.  ``window`` = None keeps every token; an integer W keeps the last W
    positions, so the cache manager may hand back pages that the window has passed.  Mixers with
    the same window share a cache group (one page pool's bookkeeping, one block table)."""

    tensors: Tuple[PagedTensor, ...]
    window: Optional[int] = None


@dataclass(frozen=True)
class KVCacheSpec:
    """The usual case of ``PagedCacheSpec``: keys ``k`` [kv_heads, page, head_dim] and values
    ``v`` transposed [kv_heads, head_dim, page] (the layout the attention kernels contract in)."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    @property
    def tensors(self) -> Tuple[PagedTensor, ...]:
        return (PagedTensor("k", (self.num_kv_heads, PAGE, self.head_dim)),
                PagedTensor("v", (self.num_kv_heads, self.head_dim, PAGE)))


@dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request (shape without the slot dimension)."""

    shape: tuple
    dtype: torch.dtype = torch.float32


# --------------------------------------------------------------------------- step context
@dataclass
class StepContext:
    """What one step's kernels need to know about the batch; built by the step function.

    Device tensors are int32.  ``T`` tokens belong to ``R`` requests; request r owns
    tokens ``q_start[r] .. q_start[r+1]``, at absolute positions
    ``kv_len[r] - q_len[r] ..  kv_len[r] - 1``.
    """

    T: int
    R: int
    dtype: torch.dtype                    # compute / activation dtype
    token_ids: torch.Tensor               # [T]
    positions: torch.Tensor               # [T] absolute position of each token
    req_of_token: torch.Tensor            # [T] row of the token's request in this step
    q_start: torch.Tensor                 # [R+1]
    kv_len: torch.Tensor                  # [R] keys visible after this step's writes
    slots: torch.Tensor                   # [R] per-request state slot
    block_tables: Dict[int, torch.Tensor]  # cache group -> [R, width] page ids (-1 = none)
    logit_rows: torch.Tensor              # [M] token rows whose logits are wanted
    # host-side copies for launch planning (never read by kernels)
    q_lens: Sequence[int] = ()
    kv_lens: Sequence[int] = ()
    max_q_len: int = 0
    max_kv_len: int = 0
    all_decode: bool = False
    host_slots: Sequence[int] = ()        # the requests' state slots, on the host
    # Set by whoever arranges the parts, for the part that runs next: it may leave its update of
    # the stream in pieces (``ops.gemm(..., may_defer=True)``) because the stream's next reader
    # adds them.  False unless an arrangement says so, so a part never defers by itself.
    may_defer: bool = False
    after_block_consumes: bool = False    # set by the model per block: whoever reads the stream after this block adds pending pieces
    workspace: Any = None                 # the runner's ops.KernelWorkspace: scratch memory of the kernels
    plans: Dict[Any, Any] = field(default_factory=dict)     # step planner -> what it made for this step
    scratch: Dict[Any, Any] = field(default_factory=dict)   # what parts share within one step; emptied per step


@dataclass
class LayerCache:
    """The view of the cache manager that one entry of the run order gets."""

    group: int = -1                       # cache group of the pages (-1: no pages)
    k: Optional[torch.Tensor] = None      # [pages, kv_heads, page_size, head_dim]   (= tensors["k"])
    v: Optional[torch.Tensor] = None      # [pages, kv_heads, head_dim, page_size]   (= tensors["v"])
    page_size: int = 0
    writes: bool = True                   # False: reads another entry's cache
    state: Optional[torch.Tensor] = None  # [max_slots, *StateSpec.shape]
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)   # every paged tensor by name: [pages, *page shape]


# --------------------------------------------------------------------------- part bases
class Part:
    """Common behaviour: declare tensors, receive them, know the compute dtype.

    ``graph_safe``: True promises that ``forward`` does the same launches, on the same addresses,
    for every step of one batch size of single tokens - it reads nothing of the step on the host
    (``ctx.host_slots``, ``ctx.q_lens``, ``ctx.kv_lens``, values of device tensors) and decides
    nothing in Python from it.  Only then may a decode step be captured once as a HIP graph and
    replayed; one part without the promise makes the whole model step eagerly.  The default is
    False: a part has to say so.
    """

    graph_safe = False

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def load(self, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        """Receive this part's tensors (relative names), already on ``device``."""
        self.dtype = dtype
        self.device = device

    def streamed_weights(self) -> List[torch.Tensor]:
        """After ``load``: the weight matrices [out, in] that this part hands to ``ops.gemm`` /
        ``ops.gemm_swiglu`` whole, in every decode step.  Whoever runs the model may keep a second
        copy of each in the order the weight-streaming kernels read (``EngineOptions.stream_copies``);
        a part that names none loses nothing but that."""
        return []


class Norm(Part):
    def forward(self, x: torch.Tensor, ctx: Optional[StepContext] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``x`` float32 [N, D] -> normalised rows in the compute dtype ([M, D] when
        ``rows`` (int32 [M]) selects rows of ``x``).  ``ctx`` is the step's context (None
        when the norm is used on its own)."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Encodes positions into queries and keys.

    ``rotary_params()`` lets the attention mixer fuse the rotation into its cache-write
    kernel; a scheme that is not a rotation returns None and implements ``apply``.
    """

    def rotary_params(self, ctx=None):
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self):
        """What the mixer keeps per request: ``KVCacheSpec`` / ``PagedCacheSpec`` (per token, in
        pages), ``StateSpec`` (fixed size), or None."""
        return None

    def step_planner(self, page_size: int):
        """Called once after ``load``.  A mixer whose kernels want host-made work lists per step
        returns a hashable *planner* with ``plan(q_lens, kv_lens) -> None | (arrays, finish)``:
        ``arrays`` are int32 numpy arrays by name, which the step function packs into its one
        upload of metadata, and ``finish(views)`` turns their device views into whatever the
        mixer reads back from ``ctx.plans[planner]``.  Planners that compare equal run once per
        step, for all their mixers.  None: nothing to plan."""
        return None

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        """Read activations ``h`` [T, D]; add the mixer's output into ``x`` (float32)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        """Read activations ``h`` [T, D]; add the result into ``x`` (float32)."""
        raise NotImplementedError


class Block(Part):
    """An arrangement of norm(s), mixer(s) and feed-forward around the residual stream.

    The stream a block receives is finished (no update pending) unless the block says that its
    first reader adds pending pieces (``reads_deferred``), and no part inside it leaves an update
    pending unless the block sets ``ctx.may_defer`` before calling it.  An arrangement that knows
    nothing of deferred updates therefore never meets one."""

    mixer: Mixer
    reads_deferred = False     # True: the block's first reader of the stream is a norm that adds pending pieces

    def mixers(self) -> List[Mixer]:
        """The block's mixers, each with a cache or state of its own.  With more than one,
        ``forward`` receives a list of ``LayerCache`` in this order instead of a single one."""
        m = getattr(self, "mixer", None)
        return [m] if m is not None else []

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------- registries
class PartRegistry:
    def __init__(self, what: str):
        self.what = what
        self._makers: Dict[str, Callable[..., Any]] = {}

    def register(self, kind: str, maker: Callable[..., Any] | None = None):
        """``register("name", cls)`` or ``@register("name")``."""
        if maker is None:
            def deco(m):
                self._makers[kind] = m
                return m
            return deco
        self._makers[kind] = maker
        return maker

    def make(self, kind: str, **params) -> Any:
        if kind not in self._makers:
            known = ", ".join(sorted(self._makers)) or "<none>"
            raise UnsupportedModelError(f"{self.what} '{kind}' is not registered (registered: {known})")
        return self._makers[kind](**params)

    def kinds(self) -> tuple:
        return tuple(sorted(self._makers))


NORMS = PartRegistry("norm")
MIXERS = PartRegistry("mixer")
FEED_FORWARDS = PartRegistry("feed-forward")
POSITION_ENCODINGS = PartRegistry("position encoding")
BLOCKS = PartRegistry("block arrangement")
