"""The step function: one batch of (request, its next tokens) through the model.

Reference: ``LLaMAModel::forward_batched(tokens, positions, seq_ids, logits)``
(src/arch/llama_model.cpp:483-605) takes flat tokens of several sequences, but rotates
every row by the first row's position and lets a portion's rows see later rows
(src/arch/transformer_block.cpp:443-444,487-509), and returns logits for all rows.  Here
each token carries its own position, sees keys at positions <= its own only, and logits
come back only for the rows asked for.

A step runs exactly the tokens it is given, as one batch, on top of the cache that earlier
steps left.  Portions of prompts and single decoded tokens mix freely.
"""
from __future__ import annotations

from dataclasses import dataclass, field
import functools
import gc
import sys
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import ops
from ..cache import CacheManager, StateSlots
from ..errors import CacheError, OutOfMemoryError, OutOfPagesError, RequestError
from ..parts import DecoderModel, LayerCache, ModelSpec, StepContext, plan_cache
from ..registry import build_model_spec, load_config
from ..weights import load_model_tensors
from .options import EngineOptions


STREAM_COPIES_MAX_SHARE = 0.5     # of the memory that is free after the weights


def stream_copies_wanted(copy_bytes: int, free_bytes: int, asked: bool) -> bool:
    """Whether a runner makes the weights' streaming copies: always when the caller asked for them
    by name (not fitting is then an ``OutOfMemoryError``); left to itself, when they take at most
    half of what is free after the weights, so that a model that fills more than a third of the
    device still loads and keeps a page pool worth having."""
    if copy_bytes <= 0:
        return False
    if asked:
        if copy_bytes > free_bytes:
            raise OutOfMemoryError(f"stream_copies=True asks for {copy_bytes / 2**30:.1f} GiB of weight copies; "
                                   f"{free_bytes / 2**30:.1f} GiB of device memory are free after the weights")
        return True
    return copy_bytes <= STREAM_COPIES_MAX_SHARE * free_bytes


def _on_own_device(method):
    """Run a runner's method with the runner's device current: kernels launch on the current
    device's stream, and a process may hold runners on several devices."""
    @functools.wraps(method)
    def wrapped(self, *args, **kwargs):
        if torch.cuda.current_device() == self.device.index:
            return method(self, *args, **kwargs)
        with torch.cuda.device(self.device):
            return method(self, *args, **kwargs)
    return wrapped


@dataclass
class StepEntry:
    """The next tokens of one live request, and which of them want logits."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()   # indices into ``tokens``


class ModelRunner:
    """Owns the model, the cache (manager + device pools + state slabs) and ``step``."""

    def __init__(self, model_dir: Optional[str], options: Optional[EngineOptions] = None, *, config=None,
                 tensors: Optional[Dict[str, torch.Tensor]] = None):
        """From a model folder, or (``model_dir`` None) from a typed config and tensors that are
        already on the device, named and shaped as the model's tensor list says."""
        self.options = options or EngineOptions()
        self.dtype = self.options.resolved_dtype()
        self.device = torch.device(self.options.device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RequestError("the engine runs on a GPU only; no CUDA/HIP device is available")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        if self.device.index >= torch.cuda.device_count():
            raise RequestError(f"device {self.options.device}: this process sees {torch.cuda.device_count()} GPU(s)")
        with torch.cuda.device(self.device):
            self._load(model_dir, config, tensors)

    def _load(self, model_dir, config, tensors) -> None:
        ops.ensure_loaded(self.dtype)
        self.config = load_config(model_dir) if model_dir is not None else config
        self.spec: ModelSpec = build_model_spec(self.config)
        if model_dir is not None:
            tensors = load_model_tensors(model_dir, self.spec.tensor_specs(), self.dtype, self.device, self.spec.ignorable)
        else:
            from ..weights.loader import check_tensors
            check_tensors({t.name: t for t in self.spec.tensor_specs()}, {n: tuple(t.shape) for n, t in tensors.items()},
                          self.spec.ignorable, "given tensors")
        if self.dtype == torch.bfloat16:
            wide = [n for n, t in tensors.items() if t.dtype == torch.float32 and t.dim() >= 2]
            if wide:
                print(f"[photon_infer_amd] {len(wide)} weight matrices are stored in 32-bit and stay so ({wide[0]}, ...): "
                      f"products with them take the float32 kernels, far slower than the bfloat16 ones; "
                      f"store the folder in bfloat16 to compute in bfloat16", file=sys.stderr, flush=True)
        self.model = DecoderModel(self.spec)
        self.model.load(tensors, self.dtype, self.device)
        del tensors
        # scratch memory of the kernels and the one residual update that may be pending: this
        # runner's own, handed to the parts with every step's context
        self.workspace = ops.KernelWorkspace(self.device)
        self.workspace.prepare(self.dtype == torch.bfloat16 and ops.fast_kernels_enabled())
        # a second copy of the matrices that every decode step streams, in the order the kernels
        # read them; made before the cache is sized, which takes what memory is left
        self.stream_copies = 0
        if self.options.stream_copies is not False and self.dtype == torch.bfloat16 and ops.fast_kernels_enabled():
            self._make_stream_copies()
        self._build_cache()
        # what the mixers want planned on the host per step (equal planners are kept once)
        self.planners = []
        for e in self.spec.run_order:
            for mixer in self.spec.layers[e.layer][1].mixers():
                planner = mixer.step_planner(self.page_size)
                if planner is not None and planner not in self.planners:
                    self.planners.append(planner)
        # a decode step is captured as a HIP graph only when every part promises that its launches
        # do not depend on host-side values of the step
        self.graph_safe = self.model.graph_safe
        self._graphs: Dict[Tuple[int, int], "_DecodeGraph"] = {}

    # ------------------------------------------------------------------ the weights' streaming copies
    def _free_device_bytes(self) -> int:
        free, _total = torch.cuda.mem_get_info(self.device)
        return free + torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)   # torch's own spare blocks

    def _make_stream_copies(self) -> None:
        """Copy the streamed matrices if that leaves room for a useful page pool
        (``stream_copies_wanted``); running out of memory on the way drops them all again.  The
        model runs without them, a little slower; only a caller who asked for them by
        ``stream_copies=True`` gets an error instead."""
        seen, mats = set(), []
        for w in self.model.streamed_weights():
            if w is not None and w.data_ptr() not in seen and ops.stream_layout_takes(w):   # a tied head names the embedding's matrix
                seen.add(w.data_ptr())
                mats.append(w)
        need = sum(w.numel() * w.element_size() for w in mats)
        asked = self.options.stream_copies is True
        if not stream_copies_wanted(need, self._free_device_bytes(), asked):
            return
        try:
            for w in mats:
                self.stream_copies += int(self.workspace.add_stream_copy(w))
        except torch.OutOfMemoryError:
            self.workspace.drop_stream_copies()
            self.stream_copies = 0
            if asked:
                raise OutOfMemoryError(f"stream_copies=True: the weights' streaming copies ({need / 2**30:.1f} GiB) "
                                       f"do not fit the device") from None
            print(f"[photon_infer_amd] no room for the weights' streaming copies ({need / 2**30:.1f} GiB): running without them",
                  file=sys.stderr, flush=True)

    # ------------------------------------------------------------------ cache set-up
    def _build_cache(self) -> None:
        o = self.options
        self.plan = plan_cache(self.spec)
        self.max_model_len = int(o.max_model_len or self.spec.max_positions)
        self.page_size = int(o.block_size)
        if self.page_size <= 0 or o.max_batch <= 0:
            raise RequestError("block_size and max_batch must be positive")
        # bytes that one page holds over all mixers that own pages (whatever each keeps per token)
        page_bytes = sum(t.page_bytes(self.page_size, self.dtype) for g in self.plan.groups for owner in g.tensors for t in owner)
        free = self._free_device_bytes()
        if o.num_blocks is not None or o.max_cache_tokens is not None:
            num_pages = int(o.num_blocks) if o.num_blocks is not None else max(1, -(-int(o.max_cache_tokens) // self.page_size))
            if num_pages <= 0:
                raise RequestError("num_blocks / max_cache_tokens must be positive")
            if num_pages * page_bytes > free:
                what = f"num_blocks={o.num_blocks}" if o.num_blocks is not None else f"max_cache_tokens={o.max_cache_tokens}"
                raise OutOfMemoryError(
                    f"{what} asks for {num_pages} pages of {page_bytes} bytes = {num_pages * page_bytes / 2**30:.1f} GiB of cache; "
                    f"{free / 2**30:.1f} GiB of device memory are free after the weights "
                    f"(at most {free // max(1, page_bytes)} pages)")
        else:
            # every slot at full length if that fits; otherwise what the given share of the free
            # memory holds, and no sequence longer than that
            wanted = max(1, -(-o.max_batch * self.max_model_len // self.page_size))
            if not 0.0 < o.memory_fraction <= 1.0:
                raise RequestError(f"memory_fraction must be in (0, 1], got {o.memory_fraction}")
            fits = int(free * o.memory_fraction) // max(1, page_bytes) if page_bytes else wanted
            num_pages = min(wanted, fits)
            if num_pages < 1:
                raise OutOfMemoryError(
                    f"no cache page of {page_bytes} bytes fits into {o.memory_fraction:.2f} of the {free / 2**30:.2f} GiB "
                    f"of device memory that are free after the weights")
            self.max_model_len = min(self.max_model_len, num_pages * self.page_size)
        self.num_pages = num_pages
        self.cache = CacheManager([g.window for g in self.plan.groups], self.page_size, num_pages,
                                  o.max_batch, self.max_model_len)
        self.states = StateSlots(self.plan.states, o.max_batch, self.device)
        # one pool per paged tensor of every mixer that owns pages, [pages, *page shape]: for
        # attention, keys [pages, kv_heads, page, head_dim] and values [pages, kv_heads, head_dim,
        # page] (the layout the kernels contract in)
        pools: Dict[tuple, Dict[str, torch.Tensor]] = {}
        try:
            for g in self.plan.groups:
                for owner, tensors in zip(g.owners, g.tensors):
                    pools[owner] = {t.name: torch.zeros((num_pages, *t.page_shape(self.page_size)), dtype=t.dtype or self.dtype,
                                                        device=self.device) for t in tensors}
        except torch.OutOfMemoryError as e:
            pools.clear()
            raise OutOfMemoryError(f"the cache pools ({num_pages} pages of {page_bytes} bytes) do not fit the device: {e}") from None
        # what each run-order entry's block is handed: its mixer's view, or a list of views when
        # the block has several mixers
        self.layer_caches: List = []
        for i, e in enumerate(self.spec.run_order):
            views = []
            for j, _mixer in enumerate(self.spec.layers[e.layer][1].mixers()):
                owner = self.plan.owner_of[(i, j)]
                lc = LayerCache(writes=e.cache_of is None, state=self.states.get(owner))
                if owner in pools:
                    lc.group = self.plan.group_of[owner]
                    lc.tensors = pools[owner]
                    lc.k, lc.v = lc.tensors.get("k"), lc.tensors.get("v")
                    lc.page_size = self.page_size
                views.append(lc)
            self.layer_caches.append(views[0] if len(views) == 1 else (views or LayerCache()))

    # ------------------------------------------------------------------ request life cycle
    def admit(self, rid: Hashable) -> int:
        slot = self.cache.admit(rid)
        self.states.clear(slot)
        return slot

    def release(self, rid: Hashable) -> None:
        self.cache.release(rid)

    # ------------------------------------------------------------------ the step
    def _check(self, entries: Sequence[StepEntry]) -> None:
        seen = set()
        vocab = self.spec.vocab_size
        for e in entries:
            if e.rid in seen:
                raise RequestError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if e.rid not in self.cache:
                raise CacheError(f"request {e.rid!r} is not live; admit it first")
            n = len(e.tokens)
            if n == 0:
                raise RequestError(f"request {e.rid!r} brings no tokens")
            if n <= 8:      # single tokens and short portions: plain comparisons beat an array round trip
                ok = all(isinstance(t, (int, np.integer)) and 0 <= t < vocab for t in e.tokens)
            else:
                arr = np.asarray(e.tokens)
                ok = arr.dtype.kind in "iu" and arr.min() >= 0 and arr.max() < vocab
            if not ok:
                bad = [t for t in e.tokens if not (isinstance(t, (int, np.integer)) and 0 <= int(t) < vocab)]
                raise RequestError(f"request {e.rid!r}: token id {bad[0]} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise RequestError(f"request {e.rid!r}: wanted row {w} is outside its {n} tokens")
            if len(e.want) > 1 and len(set(int(w) for w in e.want)) != len(e.want):
                # the final norm folds a pending update into each wanted row, one block per row
                raise RequestError(f"request {e.rid!r}: a row is wanted twice ({list(e.want)})")
            if self.cache.length(e.rid) + n > self.max_model_len:
                raise RequestError(
                    f"request {e.rid!r} would reach {self.cache.length(e.rid) + n} tokens; the limit is {self.max_model_len}")

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Pack the step's metadata, upload it in one copy, and return the views."""
        cache = self.cache
        R = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        starts = [cache.length(e.rid) for e in entries]
        kv_lens = [s + n for s, n in zip(starts, q_lens)]
        slots = [cache.slot(e.rid) for e in entries]
        T = sum(q_lens)
        q_start = np.zeros(R + 1, np.int32)
        np.cumsum(q_lens, out=q_start[1:])
        token_ids = np.concatenate([np.asarray(e.tokens, np.int32) for e in entries])
        positions = np.concatenate([np.arange(s, s + n, dtype=np.int32) for s, n in zip(starts, q_lens)])
        req_of_token = np.repeat(np.arange(R, dtype=np.int32), q_lens)
        logit_rows = np.asarray([q_start[r] + int(w) for r, e in enumerate(entries) for w in e.want], np.int32)
        width = max(1, -(-max(kv_lens) // self.page_size))
        parts = {
            "token_ids": token_ids, "positions": positions, "req_of_token": req_of_token, "q_start": q_start,
            "kv_len": np.asarray(kv_lens, np.int32), "slots": np.asarray(slots, np.int32), "logit_rows": logit_rows,
        }
        for g in range(len(cache.groups)):
            parts[f"table{g}"] = np.ascontiguousarray(cache.table_rows(g, slots, width)).reshape(-1)
        planned = []
        for i, planner in enumerate(self.planners):
            made = planner.plan(q_lens, kv_lens)
            if made is not None:
                arrays, finish = made
                parts.update({f"plan{i}.{name}": arr for name, arr in arrays.items()})
                planned.append((planner, f"plan{i}.", tuple(arrays), finish))
        views = ops.upload_arrays(parts, self.device)
        ctx = StepContext(
            T=T, R=R, dtype=self.dtype,
            token_ids=views["token_ids"], positions=views["positions"], req_of_token=views["req_of_token"],
            q_start=views["q_start"], kv_len=views["kv_len"], slots=views["slots"],
            block_tables={g: views[f"table{g}"].view(R, width) for g in range(len(cache.groups))},
            logit_rows=views["logit_rows"],
            q_lens=q_lens, kv_lens=kv_lens, max_q_len=max(q_lens), max_kv_len=max(kv_lens),
            all_decode=all(n == 1 for n in q_lens), host_slots=slots, workspace=self.workspace,
        )
        for planner, prefix, names, finish in planned:
            ctx.plans[planner] = finish({name: views[prefix + name] for name in names})
        return ctx

    def _reserve(self, entries: Sequence[StepEntry]) -> List[int]:
        """Pages for the step's new tokens: the whole step or nothing (OutOfPagesError before
        any page is taken).  Returns the requests' slots."""
        slots = [self.cache.slot(e.rid) for e in entries]
        self.cache.reserve_step(slots, [len(e.tokens) for e in entries])
        return slots

    @_on_own_device
    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits [wanted rows, vocab] on the device, in
        the order of the entries and of each entry's ``want`` (None if nothing is wanted)."""
        entries = list(entries)
        if not entries:
            return None
        self._check(entries)
        slots = self._reserve(entries)
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx, self.layer_caches)
        self.cache.commit_step(slots, [len(e.tokens) for e in entries])
        return logits

    graphs_captured = 0
    decode_logits: Optional[torch.Tensor] = None     # with options.keep_logits: the last decode step's logits [R, vocab]

    # what a caller that reads a step's tokens later needs: an event to record behind its copy
    # and page-locked memory to copy into
    def new_event(self):
        return torch.cuda.Event()

    def host_token_buffer(self, n: int) -> torch.Tensor:
        return torch.empty(n, dtype=torch.int32, pin_memory=True)

    def capture_stream(self):
        if getattr(self, "_capture_stream", None) is None:
            self._capture_stream = torch.cuda.Stream(device=self.device)
        return self._capture_stream

    def graph_pool(self):
        if getattr(self, "_graph_pool", None) is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        return self._graph_pool

    @_on_own_device
    @torch.no_grad()
    def decode_step(self, entries: Sequence[StepEntry], temperatures: Sequence[float], uniforms: Sequence[float],
                    feed: Optional[Tuple[torch.Tensor, Sequence[int]]] = None) -> torch.Tensor:
        """A batch of single tokens, one per request, each wanting its next token: the model
        and the sampling kernel run as one replayed HIP graph (captured per batch size and
        length bucket at first use) - or, when a part of the model does not promise that its
        launches are the same from step to step (``Part.graph_safe``), eagerly with the same
        kernels.  Returns the chosen token ids (int32 [R], on the device); the same buffer is
        written by the next step of the same shape, so read or copy it before launching that one.

        ``feed`` = (ids, rows): the tokens are not known on the host yet; request i's token is
        ``ids[rows[i]]``, taken on the device (``ids``: what an earlier decode_step returned).
        The entries' own token values are then ignored."""
        entries = list(entries)
        if any(len(e.tokens) != 1 for e in entries):
            raise RequestError("decode_step takes exactly one token per request")
        if feed is not None:
            if len(feed[1]) != len(entries):
                raise RequestError("decode_step: one fed row per request is needed")
            entries = [StepEntry(e.rid, [0], e.want) for e in entries]     # placeholders pass the vocabulary check
        self._check(entries)
        if not (self.graph_safe and self.options.use_graphs):
            return self._decode_eager(entries, temperatures, uniforms, feed)
        slots = self._reserve(entries)
        lengths = self.cache.lengths_of(slots)
        # one graph per batch size and length bucket: the attention kernel's key ranges follow the bucket
        bucket = ops.decode_length_bucket(int(lengths.max()) + 1)
        graph = self._graphs.get((len(entries), bucket))
        if graph is None:
            graph = self._graphs[(len(entries), bucket)] = _DecodeGraph(self, len(entries), bucket)
        out = graph.run(entries, slots, lengths, temperatures, uniforms, feed)
        self.decode_logits = graph.logits
        self.cache.commit_step(slots, [1] * len(slots))
        return out


    def _decode_eager(self, entries, temperatures, uniforms, feed) -> torch.Tensor:
        """``decode_step`` without a graph: the step function and the sampling kernel, launched
        one by one.  Parts may read the step's shape and slots on the host."""
        R = len(entries)
        entries = [StepEntry(e.rid, e.tokens, [0]) for e in entries]
        slots = self._reserve(entries)
        ctx = self.build_context(entries)
        if feed is not None:      # the tokens come from an earlier step's result, on the device
            rows = torch.tensor(list(feed[1]), dtype=torch.int32).to(self.device)
            torch.index_select(feed[0], 0, rows, out=ctx.token_ids)
        logits = self.model.forward(ctx, self.layer_caches)
        self.decode_logits = logits if self.options.keep_logits else None
        params = torch.from_numpy(np.asarray([list(temperatures), list(uniforms)], np.float32)).to(self.device)
        out = torch.empty(R, dtype=torch.int32, device=self.device)   # a buffer of its own: the step before may still be unread
        ops.sample(out, logits, params[0], params[1], ws=self.workspace)
        self.cache.commit_step(slots, [1] * R)
        return out


class _DecodeGraph:
    """The decode step of one batch size and context-length bucket as a HIP graph.

    All metadata lives in one device buffer at fixed addresses (tokens, positions, lengths,
    slots, sampling parameters, block-table rows as wide as the bucket needs); a step copies the new values
    in and replays.  Nothing in the graph depends on a host-side number: the attention grid is
    fixed by the batch size and the bucket, key ranges are derived on the device from the lengths.
    """

    def __init__(self, runner: "ModelRunner", R: int, length_bucket: int):
        self.runner, self.R = runner, R
        cache = runner.cache
        # no request of this graph is longer than the bucket: its tables need no more columns
        self.width = min(cache.max_blocks, -(-length_bucket // cache.page_size))
        G = len(cache.groups)
        names = ["token_ids", "positions", "req_of_token", "kv_len", "slots", "logit_rows", "temps", "uniforms", "feed_rows"]
        self.off, total = {}, 0
        for name in names:
            self.off[name] = (total, R)
            total += (R + 3) // 4 * 4
        self.off["q_start"] = (total, R + 1)
        total += (R + 1 + 3) // 4 * 4
        for g in range(G):
            self.off[f"table{g}"] = (total, R * self.width)
            total += (R * self.width + 3) // 4 * 4
        # two pinned staging buffers, used in turn: a step may be filled while the copy of the
        # one before it has not run yet (the engine launches one step ahead)
        self._staging = []
        for _ in range(2):
            host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
            h = {k: host[o:o + n].numpy() for k, (o, n) in self.off.items()}
            hf = {k: host[o:o + n].view(torch.float32).numpy() for k, (o, n) in self.off.items() if k in ("temps", "uniforms")}
            h["req_of_token"][:] = np.arange(R)
            h["logit_rows"][:] = np.arange(R)
            h["q_start"][:] = np.arange(R + 1)
            self._staging.append((host, h, hf))
        self._copied = [torch.cuda.Event(), torch.cuda.Event()]    # a staging buffer's last copy to the device
        self._turn = 0
        self.host, self.h, self.hf = self._staging[0]
        self.dev = torch.zeros(total, dtype=torch.int32, device=runner.device)
        d = {k: self.dev[o:o + n] for k, (o, n) in self.off.items()}
        self.ctx = StepContext(
            T=R, R=R, dtype=runner.dtype, token_ids=d["token_ids"], positions=d["positions"],
            req_of_token=d["req_of_token"], q_start=d["q_start"], kv_len=d["kv_len"], slots=d["slots"],
            block_tables={g: d[f"table{g}"].view(R, self.width) for g in range(G)}, logit_rows=d["logit_rows"],
            q_lens=[1] * R, kv_lens=(), max_q_len=1, max_kv_len=length_bucket, all_decode=True,
            workspace=runner.workspace)
        self.feed_rows = d["feed_rows"]
        self.temps = d["temps"].view(torch.float32)
        self.uniforms = d["uniforms"].view(torch.float32)
        self.sampled = torch.zeros(R, dtype=torch.int32, device=runner.device)
        self.logits: Optional[torch.Tensor] = None
        self.graph: Optional[torch.cuda.CUDAGraph] = None

    def _fill(self, entries, slots, lengths, temperatures, uniforms, feed) -> None:
        cache = self.runner.cache
        self._turn ^= 1
        self.host, self.h, self.hf = self._staging[self._turn]
        self._copied[self._turn].synchronize()      # a caller more than one step ahead waits here, not corrupts
        if feed is None:
            self.h["token_ids"][:] = [e.tokens[0] for e in entries]
        else:
            self.h["feed_rows"][:] = feed[1]
        self.h["positions"][:] = lengths
        self.h["kv_len"][:] = lengths + 1
        self.h["slots"][:] = slots
        self.hf["temps"][:] = temperatures
        self.hf["uniforms"][:] = uniforms
        for g in range(len(cache.groups)):
            self.h[f"table{g}"].reshape(self.R, self.width)[:] = cache.table_rows(g, slots, self.width)
        self.ctx.host_slots = slots
        self.dev.copy_(self.host, non_blocking=True)
        self._copied[self._turn].record()
        if feed is not None:      # the tokens come from an earlier step's result, on the device
            torch.index_select(feed[0], 0, self.feed_rows, out=self.ctx.token_ids)

    def _body(self) -> None:
        logits = self.runner.model.forward(self.ctx, self.runner.layer_caches)
        ops.sample(self.sampled, logits, self.temps, self.uniforms, ws=self.runner.workspace)
        # kept alive, the logits stay where every replay writes them (and the pool cannot give
        # their memory to another graph); otherwise a graph holds nothing between replays
        self.logits = logits if self.runner.options.keep_logits else None

    def run(self, entries, slots, lengths, temperatures, uniforms, feed=None) -> torch.Tensor:
        self._fill(entries, slots, lengths, temperatures, uniforms, feed)
        if self.graph is None:
            runner = self.runner
            # The runner's very first decode step runs eagerly, so that everything made at first
            # use (workspaces, kernel libraries) exists before any capture; it does the step's
            # work, and the capture that follows only records.  Every later graph is captured
            # straight away and replayed for its first step.
            eager_first = not runner.graphs_captured
            first_logits = None
            if eager_first:
                self._body()
                first_logits = self.logits
                torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # no garbage collection while the stream is capturing: a collected tensor of some
            # earlier engine (pinned memory, events) would make calls that a capture forbids
            collecting = gc.isenabled()
            gc.disable()
            try:
                # Capture on a stream of the runner's own (default priority), begun and ended by
                # hand: no device-wide wait, collection or cache flush per graph.  All graphs
                # of a runner take their intermediate buffers from one pool: they never run at
                # the same time and hold nothing in it between replays (the sampled tokens and
                # the metadata lie outside).
                side, main = runner.capture_stream(), torch.cuda.current_stream()
                side.wait_stream(main)
                with torch.cuda.stream(side):
                    graph.capture_begin(pool=runner.graph_pool())
                    try:
                        self._body()
                    finally:
                        graph.capture_end()
                main.wait_stream(side)
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
            runner.graphs_captured += 1
            if not eager_first:
                graph.replay()
            elif first_logits is not None:
                self.logits.copy_(first_logits)      # the capture recorded only: this step's logits are the eager run's
        else:
            self.graph.replay()
        return self.sampled
