"""Requests and the continuous-batching scheduler.

Reference: include/photon/scheduler/inference_request.hpp (states WAITING / RUNNING /
PREEMPTED / FINISHED, ``num_computed_tokens`` as the resume point) and
include/photon/scheduler/continuous_batch_scheduler.hpp:133-158 (two phases per step:
every running request continues, then waiting requests are admitted first come first
served).  Kept: the states, the two phases, the chunk size, the names.  Changed:

* a token budget per step: requests with one token left to feed (decodes) go first, then
  running prompts, then admissions, each prompt getting
  ``min(chunk_size, remaining, budget left)`` tokens - so portions vary in size;
* the portion that ends a request's known tokens is sampled in the same step; the
  reference feeds the last prompt token a second time instead
  (include/photon/scheduler/inference_request.hpp:208-219);
* admission asks for a free slot and for pages for the first portion; the reference counts
  waiting requests against ``max_sequences`` (continuous_batch_scheduler.hpp:143,202-204)
  and reserves a request's whole lifetime of pages up front;
* when a running request cannot get its next page, the most recently admitted running
  request is preempted (the reference declares PREEMPTED but never enters it): its pages
  and slot are given back, it returns to the front of the waiting queue and is recomputed
  from its prompt plus what it has generated.  A request that cannot fit even alone is
  finished with reason "out_of_pages".
"""
from __future__ import annotations

import enum
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..errors import RequestError
from ..sampling.sampler import SamplingParams


class RequestState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    PREEMPTED = "preempted"


class InferenceRequest:
    """One generation request; mirrors include/photon/scheduler/inference_request.hpp:50-320."""

    def __init__(self, request_id: int, prompt_tokens: Sequence[int], params: SamplingParams, prompt: str = ""):
        self.request_id = request_id
        self.prompt = prompt
        self.prompt_tokens: List[int] = [int(t) for t in prompt_tokens]
        self._prompt_len = len(self.prompt_tokens)
        self.params = params
        self.state = RequestState.WAITING
        self.num_computed_tokens = 0
        self.generated_tokens: List[int] = []
        self.finish_reason: Optional[str] = None
        self.num_preemptions = 0
        self.arrival_time = time.perf_counter()
        self.start_time: Optional[float] = None
        self.finish_time: Optional[float] = None

    # ---- sizes
    @property
    def max_new_tokens(self) -> int:
        return self.params.max_new_tokens

    def prompt_len(self) -> int:
        return len(self.prompt_tokens)

    def num_generated(self) -> int:
        return len(self.generated_tokens)

    def total_tokens(self) -> int:
        return self._prompt_len + len(self.generated_tokens)

    def all_tokens(self) -> List[int]:
        return self.prompt_tokens + self.generated_tokens

    def remaining(self) -> int:
        """Known tokens that have not been fed through the model yet (>= 1 while running)."""
        return self._prompt_len + len(self.generated_tokens) - self.num_computed_tokens

    # ---- phases (a request that was preempted is a prompt again)
    def is_finished(self) -> bool:
        return self.state is RequestState.FINISHED

    def is_prefill(self) -> bool:
        return self.remaining() > 1 or not self.generated_tokens

    def is_decode(self) -> bool:
        return (self.state is not RequestState.FINISHED and bool(self.generated_tokens)
                and self._prompt_len + len(self.generated_tokens) - self.num_computed_tokens == 1)

    def next_tokens(self, n: int) -> List[int]:
        c = self.num_computed_tokens
        if c >= len(self.prompt_tokens):
            return self.generated_tokens[c - len(self.prompt_tokens): c - len(self.prompt_tokens) + n]
        return self.all_tokens()[c:c + n]

    def current_position(self) -> int:
        return self.num_computed_tokens

    # ---- transitions
    def start_running(self) -> None:
        self.state = RequestState.RUNNING
        if self.start_time is None:
            self.start_time = time.perf_counter()

    def finish(self, reason: str) -> None:
        self.state = RequestState.FINISHED
        self.finish_reason = reason
        self.finish_time = time.perf_counter()

    def preempt(self) -> None:
        self.state = RequestState.PREEMPTED
        self.num_computed_tokens = 0
        self.num_preemptions += 1

    def resume(self) -> None:
        self.state = RequestState.WAITING

    def add_computed_tokens(self, count: int) -> None:
        self.num_computed_tokens += count

    def add_token(self, token: int, eos_token_ids: Sequence[int], max_model_len: int) -> bool:
        """Append a sampled token; returns False when the request is finished by it
        (include/photon/scheduler/inference_request.hpp:172-182; the end token is kept)."""
        self.generated_tokens.append(int(token))
        if not self.params.ignore_eos and int(token) in eos_token_ids:
            self.finish("eos")
        elif self.num_generated() >= self.max_new_tokens:
            self.finish("length")
        elif self.total_tokens() > max_model_len:
            self.finish("max_model_len")  # the new token could not be fed any more
        return not self.is_finished()

    # ---- timing
    def latency_seconds(self) -> float:
        return (self.finish_time or time.perf_counter()) - self.arrival_time

    def execution_time_seconds(self) -> float:
        if self.start_time is None:
            return 0.0
        return (self.finish_time or time.perf_counter()) - self.start_time


@dataclass
class ScheduledBatch:
    """What one step runs: (request, number of its next tokens) pairs."""

    items: List[Tuple[InferenceRequest, int]] = field(default_factory=list)
    preempted: List[InferenceRequest] = field(default_factory=list)
    finished: List[InferenceRequest] = field(default_factory=list)   # ended without running (out of pages)

    @property
    def requests(self) -> List[InferenceRequest]:
        return [r for r, _ in self.items]

    def batch_size(self) -> int:
        return len(self.items)

    def num_tokens(self) -> int:
        return sum(n for _, n in self.items)

    def empty(self) -> bool:
        return not self.items


@dataclass
class SchedulerStats:
    num_running: int = 0
    num_waiting: int = 0
    num_finished: int = 0
    total_requests: int = 0
    num_preemptions: int = 0
    num_aborted: int = 0
    num_steps: int = 0
    tokens_scheduled: int = 0


class ContinuousBatchScheduler:
    def __init__(self, cache, max_batch_size: int, max_step_tokens: int, chunk_size: int = 256,
                 max_model_len: Optional[int] = None, owner=None):
        """``cache``: the CacheManager (asked about pages and slots).  ``owner``: whoever
        admits and releases requests in it (defaults to the manager itself; the engine
        passes its runner so that per-request state is cleared on admission)."""
        if max_batch_size <= 0 or max_step_tokens <= 0 or chunk_size <= 0:
            raise RequestError("max_batch_size, max_step_tokens and chunk_size must be positive")
        self.cache = cache
        self.owner = owner if owner is not None else cache
        self.max_batch_size = int(max_batch_size)
        self.max_step_tokens = int(max_step_tokens)
        self.chunk_size = int(chunk_size)
        self.max_model_len = int(max_model_len or cache.max_model_len)
        self.waiting: Deque[InferenceRequest] = deque()
        self.running: List[InferenceRequest] = []        # in admission order
        self.requests: Dict[int, InferenceRequest] = {}
        self._next_id = 0
        self._preemptions = 0
        self._aborted = 0
        self._steps = 0
        self._tokens = 0

    # ------------------------------------------------------------------ intake
    def add_request(self, prompt_tokens: Sequence[int], params: Optional[SamplingParams] = None,
                    prompt: str = "") -> int:
        params = params or SamplingParams()
        if len(prompt_tokens) == 0:
            raise RequestError("a request needs at least one prompt token")
        if len(prompt_tokens) > self.max_model_len:
            raise RequestError(
                f"prompt of {len(prompt_tokens)} tokens is longer than max_model_len {self.max_model_len}")
        if params.max_new_tokens <= 0:
            raise RequestError("max_new_tokens must be positive")
        rid = self._next_id
        self._next_id += 1
        req = InferenceRequest(rid, prompt_tokens, params, prompt)
        self.waiting.append(req)
        self.requests[rid] = req
        return rid

    # ------------------------------------------------------------------ one step's decisions
    def _fits(self, need: Sequence[int], held: Sequence[int]) -> bool:
        for g, n in enumerate(need):
            if n and n > self.cache.free_pages(g) - held[g]:
                return False
        return True

    def _preempt(self, victim: InferenceRequest, batch: ScheduledBatch, held: List[int]) -> None:
        for i, (r, n) in enumerate(batch.items):
            if r is victim:  # it was already in this step: give back what was promised to it
                for g, p in enumerate(self.cache.pages_needed(r.request_id, n)):
                    held[g] -= p
                del batch.items[i]
                break
        self.owner.release(victim.request_id)
        self.running.remove(victim)
        victim.preempt()
        victim.resume()
        self.waiting.appendleft(victim)
        batch.preempted.append(victim)
        self._preemptions += 1

    def schedule_next_batch(self) -> ScheduledBatch:
        batch = ScheduledBatch()
        budget = self.max_step_tokens
        held = [0] * len(self.cache.groups)

        # Phase 1: running requests; those with a single token to feed first
        decoding = [r.is_decode() for r in self.running]
        order = None
        if self.running and all(decoding) and budget >= len(self.running):
            # the common step: everyone decodes; one question for all of them
            need = self.cache.pages_needed_step([r.request_id for r in self.running], [1] * len(self.running))
            if self._fits(need, held):
                held = list(need)
                batch.items = [(r, 1) for r in self.running]
                budget -= len(self.running)
                order = []
        if order is None:
            order = [r for r, d in zip(self.running, decoding) if d] + [r for r, d in zip(self.running, decoding) if not d]
        for req in order:
            if req not in self.running:      # preempted while serving an earlier one
                continue
            if budget <= 0:
                break
            n = min(req.remaining(), self.chunk_size, budget)
            while True:
                need = self.cache.pages_needed(req.request_id, n)
                if self._fits(need, held):
                    for g, p in enumerate(need):
                        held[g] += p
                    batch.items.append((req, n))
                    budget -= n
                    break
                victim = self.running[-1]
                if victim is req and len(self.running) == 1:
                    # alone and still too big for the pool: it can never run
                    self.owner.release(req.request_id)
                    self.running.remove(req)
                    req.finish("out_of_pages")
                    batch.finished.append(req)
                    break
                self._preempt(victim, batch, held)
                if victim is req:
                    break

        # Phase 2: admit waiting requests, first come first served, while there is room
        while self.waiting and budget > 0 and len(self.running) < self.max_batch_size and self.cache.free_slots > 0:
            req = self.waiting[0]
            if req in batch.preempted:       # do not bounce a request within one step
                break
            n = min(req.remaining(), self.chunk_size, budget)
            need = self.cache.pages_needed(None, n)
            # room for everything the request already brings (its prompt, and what it generated
            # before a preemption), not only for this portion: admitting on the first portion
            # alone lets requests in that are preempted again before their prompt is through
            if not self._fits(self.cache.pages_needed(None, req.remaining()), held):
                if not self.running and not batch.items:
                    # nothing else holds pages: this request can never start
                    self.waiting.popleft()
                    req.finish("out_of_pages")
                    batch.finished.append(req)
                    continue
                break
            self.waiting.popleft()
            self.owner.admit(req.request_id)
            req.start_running()
            self.running.append(req)
            for g, p in enumerate(need):
                held[g] += p
            batch.items.append((req, n))
            budget -= n

        self._steps += 1
        self._tokens += batch.num_tokens()
        return batch

    def note_step(self, tokens: int) -> None:
        """A step that was launched without asking (the engine's step ahead) counts too."""
        self._steps += 1
        self._tokens += tokens

    def abort(self, request_id: int) -> bool:
        """Cancel a request wherever it is: a waiting one leaves the queue, a running one gives its
        slot and pages back at once.  It ends with ``finish_reason = "aborted"`` and keeps what it
        has generated.  False: unknown or already finished.  (The reference frees only on finish,
        include/photon/scheduler/continuous_batch_scheduler.hpp:169-182.)"""
        req = self.requests.get(request_id)
        if req is None or req.is_finished():
            return False
        if req in self.running:
            self.running.remove(req)
            self.owner.release(req.request_id)
        else:
            self.waiting.remove(req)
        req.finish("aborted")
        self._aborted += 1
        return True

    def update_after_step(self, finished: Sequence[InferenceRequest]) -> None:
        """Requests that ended in this step leave the running list and the cache."""
        for req in finished:
            if req in self.running:
                self.running.remove(req)
                self.owner.release(req.request_id)

    # ------------------------------------------------------------------ queries
    def get_request(self, request_id: int) -> Optional[InferenceRequest]:
        return self.requests.get(request_id)

    def has_work(self) -> bool:
        return bool(self.running or self.waiting)

    def num_running(self) -> int:
        return len(self.running)

    def num_waiting(self) -> int:
        return len(self.waiting)

    def get_stats(self) -> SchedulerStats:
        return SchedulerStats(
            num_running=len(self.running), num_waiting=len(self.waiting),
            num_finished=sum(r.is_finished() for r in self.requests.values()),
            total_requests=len(self.requests), num_preemptions=self._preemptions, num_aborted=self._aborted,
            num_steps=self._steps, tokens_scheduled=self._tokens)

    def clear_finished_requests(self) -> None:
        for rid in [rid for rid, r in self.requests.items() if r.is_finished()]:
            del self.requests[rid]
