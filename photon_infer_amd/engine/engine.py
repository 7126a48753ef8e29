"""The engine: requests in, tokens out, by continuous batching over ``ModelRunner.step``.

Reference: ``ContinuousBatchEngine`` (include/photon/scheduler/continuous_batch_engine.hpp:48-315):
``add_request`` -> ``run_until_complete`` (loop: ``schedule_next_batch`` ->
``execute_batch_step``) -> ``get_result``.  The same names and meanings are kept; requests
are given as token ids (text goes through the tokenizer of the command line).
"""
from __future__ import annotations

import sys
import time
from typing import Dict, List, Optional, Sequence

import torch

from ..errors import RequestError
from ..sampling import Sampler, SamplingParams, uniform_draw
from .options import EngineOptions
from .scheduler import ContinuousBatchScheduler, InferenceRequest, ScheduledBatch, SchedulerStats
from .step import ModelRunner, StepEntry


class _InFlight:
    """A decode step that runs on the GPU while the host goes on."""

    def __init__(self, reqs: List[InferenceRequest], ids, host, done):
        self.reqs = reqs            # in the order of the step's rows
        self.ids = ids              # the step's tokens on the device
        self.host = host            # pinned buffer they are copied to
        self.done = done            # event recorded behind the copy
        self.ended: List[InferenceRequest] = []   # requests in this step that had already ended when it was launched


class ContinuousBatchEngine:
    def __init__(self, model_dir: Optional[str], options: Optional[EngineOptions] = None, *,
                 runner: Optional[ModelRunner] = None, **option_fields):
        """``ContinuousBatchEngine(model_dir, dtype="bfloat16", max_batch=64, ...)``: any field
        of EngineOptions may be given by keyword.  ``runner``: use a ModelRunner that already
        holds the model (then ``model_dir`` is None and the runner's options apply)."""
        if runner is not None:
            options = runner.options
        elif options is None:
            options = EngineOptions(**option_fields)
        elif option_fields:
            raise RequestError("give either an EngineOptions object or option fields, not both")
        self.options = options
        self.runner = runner if runner is not None else ModelRunner(model_dir, options)
        self.scheduler = ContinuousBatchScheduler(
            self.runner.cache, options.max_batch, options.max_step_tokens, options.chunk_size,
            self.runner.max_model_len, owner=self.runner)
        self.sampler = Sampler(self.runner.device, self.runner.workspace)
        self.eos_token_ids = tuple(self.runner.spec.eos_token_ids)
        self.steps = 0
        self.host_wait_seconds = 0.0     # time the host spent waiting for the GPU's tokens
        # a decode step that was launched and whose tokens have not been read yet
        self._in_flight: Optional[_InFlight] = None
        # pinned buffers the sampled tokens are copied to, by (batch size, turn)
        self._buffers: Dict[tuple, "torch.Tensor"] = {}

    @property
    def config(self):
        return self.runner.config

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt_tokens: Sequence[int], max_new_tokens: int = 128, temperature: float = 0.0,
                    seed: Optional[int] = None, ignore_eos: bool = False, prompt: str = "") -> int:
        vocab = self.runner.spec.vocab_size
        for t in prompt_tokens:
            if not 0 <= int(t) < vocab:
                raise RequestError(f"token id {t} is outside the vocabulary of {vocab}")
        params = SamplingParams(temperature=float(temperature), max_new_tokens=int(max_new_tokens),
                                seed=-1 if seed is None else int(seed), ignore_eos=ignore_eos)
        rid = self.scheduler.add_request(prompt_tokens, params, prompt)
        if seed is None:  # a stream of its own, fixed by the engine's seed and the request's number
            params.seed = (self.options.seed * 1_000_003 + rid) & 0x7FFFFFFFFFFFFFFF
        return rid

    def get_request(self, request_id: int) -> Optional[InferenceRequest]:
        return self.scheduler.get_request(request_id)

    def get_result(self, request_id: int) -> List[int]:
        """Generated token ids of a finished request (empty while it is unfinished)."""
        req = self.scheduler.get_request(request_id)
        if req is None or not req.is_finished():
            return []
        return list(req.generated_tokens)

    def get_stats(self) -> SchedulerStats:
        return self.scheduler.get_stats()

    def abort(self, request_id: int) -> bool:
        """Cancel a request: waiting, running, or in a decode step that was launched and has not
        been read yet.  Its slot and pages are free when the call returns (a step already launched
        may still write the request's last token into them; whatever is given these pages next is
        launched after it on the same stream), the token of a launched step is dropped, and the
        request ends with ``finish_reason == "aborted"`` holding what it had generated.  Returns
        False for a request that is unknown or already finished."""
        req = self.scheduler.get_request(request_id)
        if req is None or not self.scheduler.abort(request_id):
            return False
        fl = self._in_flight
        if fl is not None and req in fl.reqs and req not in fl.ended:
            fl.ended.append(req)          # its row of the launched step is read past, and it is in no later step
        return True

    # ------------------------------------------------------------------ running
    def step(self) -> List[InferenceRequest]:
        """Schedule and run one batch; returns the requests known to have finished by the end of
        the call.  With ``lookahead`` a decode step's tokens are read during the next call: the
        step after it is launched first, from what is certain without them."""
        device = self.runner.device
        if getattr(device, "type", None) == "cuda" and torch.cuda.current_device() != device.index:
            with torch.cuda.device(device):      # a process may hold engines on several devices
                return self._step()
        return self._step()

    def _step(self) -> List[InferenceRequest]:
        if self._in_flight is not None:
            return self._step_ahead()
        batch = self.scheduler.schedule_next_batch()
        finished = list(batch.finished)
        if batch.empty():
            return finished
        finished += self.execute_batch_step(batch)
        return finished

    # ---- one step ahead
    def _launch_decode(self, reqs: List[InferenceRequest], feed=None, pending: int = 0) -> None:
        """Launch a decode step for ``reqs`` and start the copy of its tokens to the host.
        ``pending``: tokens of each request that are sampled but not yet known here (0 or 1)."""
        entries = [StepEntry(r.request_id, r.next_tokens(1) if feed is None else [0], [0]) for r in reqs]
        temps = [r.params.temperature for r in reqs]
        draws = [uniform_draw(r.params.seed, r.num_generated() + pending) if r.params.temperature > 0 else 0.0 for r in reqs]
        ids = self.runner.decode_step(entries, temps, draws, feed)
        fl = _InFlight(reqs, ids, self._token_buffer(len(reqs)), self.runner.new_event())
        fl.host.copy_(ids, non_blocking=True)
        fl.done.record()
        self._in_flight = fl
        self.steps += 1

    def _token_buffer(self, n: int):
        # two pinned buffers per size, used in turn: one is still being read when the next copy starts
        key = (n, self.steps % 2)
        buf = self._buffers.get(key)
        if buf is None:
            buf = self._buffers[key] = self.runner.host_token_buffer(n)
        return buf

    def _collect(self, fl: "_InFlight", skip: Sequence[InferenceRequest] = ()) -> List[InferenceRequest]:
        """Read a launched step's tokens and book them; returns the requests they finished."""
        t0 = time.perf_counter()
        fl.done.synchronize()
        self.host_wait_seconds += time.perf_counter() - t0
        done = []
        for req, tok in zip(fl.reqs, fl.host.tolist()):
            if req in skip:            # ended a step earlier; this token was computed for nothing
                continue
            req.add_computed_tokens(1)
            if not req.add_token(tok, self.eos_token_ids, self.runner.max_model_len):
                done.append(req)
        return done

    def _step_ahead(self) -> List[InferenceRequest]:
        fl, self._in_flight = self._in_flight, None
        sched = self.scheduler
        # who certainly goes on after the step in flight: everyone it does not end by length.
        # An end token would end one more, which is only known once the tokens are here.
        nxt = [r for r in fl.reqs if r not in fl.ended and r.num_generated() + 1 < r.max_new_tokens
               and r.total_tokens() + 1 <= self.runner.max_model_len]
        # only when the step in flight is all there is to run (nobody waits, nobody else runs),
        # the token budget allows it and every next page is there; otherwise the scheduler decides
        ahead = (bool(nxt) and not sched.waiting and len(sched.running) == len(fl.reqs)
                 and len(nxt) <= sched.max_step_tokens
                 and all(n <= self.runner.cache.free_pages(g)
                         for g, n in enumerate(self.runner.cache.pages_needed_step([r.request_id for r in nxt], [1] * len(nxt)))))
        if ahead:
            rows = [fl.reqs.index(r) for r in nxt] if len(nxt) != len(fl.reqs) else list(range(len(nxt)))
            self._launch_decode(nxt, feed=(fl.ids, rows), pending=1)
            sched.note_step(len(nxt))
        done = self._collect(fl, skip=fl.ended)
        if self._in_flight is not None:
            # requests that an end token finished are in the step just launched: they leave when it is read
            self._in_flight.ended = [r for r in done if r in self._in_flight.reqs]
            sched.update_after_step([r for r in done if r not in self._in_flight.reqs] + list(fl.ended))
        else:
            sched.update_after_step(done + list(fl.ended))
        return done

    def execute_batch_step(self, batch: ScheduledBatch) -> List[InferenceRequest]:
        entries, sampled_reqs = [], []
        for req, n in batch.items:
            ends = req.num_computed_tokens + n == req.total_tokens()
            entries.append(StepEntry(req.request_id, req.next_tokens(n), [n - 1] if ends else []))
            if ends:
                sampled_reqs.append(req)
        temps = [r.params.temperature for r in sampled_reqs]
        draws = [uniform_draw(r.params.seed, r.num_generated()) if r.params.temperature > 0 else 0.0
                 for r in sampled_reqs]
        tokens: List[int] = []
        if self.options.use_graphs and len(sampled_reqs) == len(entries) and all(n == 1 for _, n in batch.items):
            # single tokens only, every one sampled: the replayed graph (model + sampling kernel), or
            # the same launched one by one when a part of the model does not allow a graph
            if self.options.lookahead:
                self._launch_decode(sampled_reqs)
                return []                   # its tokens are read in the next call
            ids = self.runner.decode_step(entries, temps, draws)
            t0 = time.perf_counter()
            tokens = ids.tolist()
            self.host_wait_seconds += time.perf_counter() - t0
        else:
            logits = self.runner.step(entries)
            if sampled_reqs:
                t0 = time.perf_counter()
                tokens = self.sampler.sample(logits, temps, draws)
                self.host_wait_seconds += time.perf_counter() - t0
        done = []
        for req, n in batch.items:
            req.add_computed_tokens(n)
        for req, tok in zip(sampled_reqs, tokens):
            if not req.add_token(tok, self.eos_token_ids, self.runner.max_model_len):
                done.append(req)
        self.scheduler.update_after_step(done)
        self.steps += 1
        return done

    def has_work(self) -> bool:
        """Requests waiting or running, or a launched step whose tokens have not been read."""
        return self.scheduler.has_work() or self._in_flight is not None

    def run_until_complete(self, print_progress: bool = False) -> None:
        while self.has_work():
            if print_progress and self.steps % 10 == 0:
                s = self.scheduler.get_stats()
                print(f"Step {self.steps}: Running={s.num_running} Waiting={s.num_waiting} Finished={s.num_finished}",
                      file=sys.stderr, flush=True)
            self.step()
        if print_progress:
            s = self.scheduler.get_stats()
            print(f"Complete! Total steps: {self.steps} Total requests: {s.total_requests}", file=sys.stderr, flush=True)

    # ------------------------------------------------------------------ convenience
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128, temperature: float = 0.0,
                 seed: Optional[int] = None, ignore_eos: bool = False) -> List[List[int]]:
        """Generate for every prompt (token id lists); returns the new token ids of each."""
        ids = [self.add_request(p, max_new_tokens, temperature,
                                None if seed is None else seed + i, ignore_eos) for i, p in enumerate(prompts)]
        self.run_until_complete()
        return [self.get_result(i) for i in ids]


Engine = ContinuousBatchEngine
