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
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from ..cache import CacheManager, StateSlots
from ..errors import CacheError, RequestError
from ..parts import DecoderModel, LayerCache, ModelSpec, StepContext, plan_cache
from ..registry import build_model_spec, load_config
from ..weights import load_model_tensors
from .options import EngineOptions


@dataclass
class StepEntry:
    """The next tokens of one live request, and which of them want logits."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()   # indices into ``tokens``


class ModelRunner:
    """Owns the model, the cache (manager + device pools + state slabs) and ``step``."""

    def __init__(self, model_dir: str, options: Optional[EngineOptions] = None):
        self.options = options or EngineOptions()
        self.dtype = self.options.resolved_dtype()
        self.device = torch.device(self.options.device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RequestError("the engine runs on a GPU only; no CUDA/HIP device is available")
        ops.ensure_loaded(self.dtype)
        self.config = load_config(model_dir)
        self.spec: ModelSpec = build_model_spec(self.config)
        tensors = load_model_tensors(model_dir, self.spec.tensor_specs(), self.dtype, self.device, self.spec.ignorable)
        self.model = DecoderModel(self.spec)
        self.model.load(tensors, self.dtype, self.device)
        del tensors
        self._build_cache()

    # ------------------------------------------------------------------ cache set-up
    def _build_cache(self) -> None:
        o = self.options
        self.plan = plan_cache(self.spec)
        self.max_model_len = int(o.max_model_len or self.spec.max_positions)
        self.page_size = int(o.block_size)
        if o.num_blocks is not None:
            num_pages = int(o.num_blocks)
        else:
            tokens = o.max_cache_tokens if o.max_cache_tokens is not None else o.max_batch * self.max_model_len
            num_pages = max(1, -(-int(tokens) // self.page_size))
        self.num_pages = num_pages
        self.cache = CacheManager([g.window for g in self.plan.groups], self.page_size, num_pages,
                                  o.max_batch, self.max_model_len)
        self.states = StateSlots(self.plan.states, o.max_batch, self.device)
        # one K and one V pool per run-order entry that owns pages: keys [pages, kv_heads, page,
        # head_dim], values [pages, kv_heads, head_dim, page] (the layout the kernels contract in)
        pools: Dict[int, tuple] = {}
        for g in self.plan.groups:
            for entry, (nkv, hd) in zip(g.entries, g.kv_shapes):
                pools[entry] = (torch.zeros((num_pages, nkv, self.page_size, hd), dtype=self.dtype, device=self.device),
                                torch.zeros((num_pages, nkv, hd, self.page_size), dtype=self.dtype, device=self.device))
        self.layer_caches: List[LayerCache] = []
        for i, e in enumerate(self.spec.run_order):
            owner = i if e.cache_of is None else e.cache_of
            lc = LayerCache(writes=e.cache_of is None, state=self.states.get(owner))
            if owner in pools:
                lc.group = self.plan.group_of_entry[owner]
                lc.k, lc.v = pools[owner]
                lc.page_size = self.page_size
            self.layer_caches.append(lc)

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
            bad = [t for t in e.tokens if not 0 <= int(t) < vocab]
            if bad:
                raise RequestError(f"request {e.rid!r}: token id {bad[0]} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise RequestError(f"request {e.rid!r}: wanted row {w} is outside its {n} tokens")
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
        extra = ops.plan_attention(q_lens, kv_lens, self.dtype) if T else {}
        parts.update(extra.get("arrays", {}))
        views = _upload(parts, self.device)
        ctx = StepContext(
            T=T, R=R, dtype=self.dtype,
            token_ids=views["token_ids"], positions=views["positions"], req_of_token=views["req_of_token"],
            q_start=views["q_start"], kv_len=views["kv_len"], slots=views["slots"],
            block_tables={g: views[f"table{g}"].view(R, width) for g in range(len(cache.groups))},
            logit_rows=views["logit_rows"],
            q_lens=q_lens, kv_lens=kv_lens, max_q_len=max(q_lens), max_kv_len=max(kv_lens),
            all_decode=all(n == 1 for n in q_lens), host_slots=slots,
        )
        ops.attach_attention_plan(ctx, extra, views)
        return ctx

    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits [wanted rows, vocab] on the device, in
        the order of the entries and of each entry's ``want`` (None if nothing is wanted)."""
        entries = list(entries)
        if not entries:
            return None
        self._check(entries)
        # pages for the new tokens: refuse the whole step before taking any page
        held = [0] * len(self.cache.groups)
        for e in entries:
            need = self.cache.pages_needed(e.rid, len(e.tokens))
            held = [h + n for h, n in zip(held, need)]
        for g, h in enumerate(held):
            if h > self.cache.free_pages(g):
                from ..errors import OutOfPagesError
                raise OutOfPagesError(
                    f"the step needs {h} more pages in cache group {g}, {self.cache.free_pages(g)} are free")
        for e in entries:
            self.cache.reserve(e.rid, len(e.tokens))
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx, self.layer_caches)
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
        return logits


def _upload(parts: Dict[str, np.ndarray], device) -> Dict[str, torch.Tensor]:
    """Concatenate int32 arrays (each padded to 16 bytes), copy once, return device views."""
    offsets, total = {}, 0
    for name, arr in parts.items():
        offsets[name] = (total, arr.size)
        total += (arr.size + 3) // 4 * 4
    packed = np.zeros(max(total, 4), np.int32)
    for name, arr in parts.items():
        o, n = offsets[name]
        packed[o:o + n] = arr
    dev = torch.from_numpy(packed).to(device)
    return {name: dev[o:o + n] for name, (o, n) in offsets.items()}
