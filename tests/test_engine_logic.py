"""The engine's bookkeeping without a GPU: ``ContinuousBatchEngine`` over a runner that computes
nothing.  The stand-in keeps what a real runner keeps (the page pool, the cache's lengths, one
result buffer per batch size that the next step of that size overwrites) and answers every step
with a token that is a fixed function of the request's whole token history and its draw, so the
right answer of any request is known without the engine: whatever the scheduler cuts, batches,
preempts, launches a step ahead or aborts, the tokens must be those of the request run alone.
Random workloads: arrivals while others run, pools so small that requests are preempted, end
tokens that end a request while it is already in the step launched ahead, aborts at any time.
"""
import random
import types

import pytest
import torch

from photon_infer_amd.cache import CacheManager
from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions, StepEntry
from photon_infer_amd.errors import RequestError
from photon_infer_amd.sampling import uniform_draw

VOCAB = 97
END = 7


def token_after(history, draw: float) -> int:
    """The stand-in model and sampler in one: any function of all tokens so far and the draw."""
    h = 1469598103934665603
    for t in history:
        h = ((h ^ (int(t) + 1)) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    h ^= int(draw * (1 << 24))
    h = (h * 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
    return (h >> 33) % VOCAB


def alone(prompt, max_new, temperature, seed, ignore_eos, max_model_len):
    """What the request generates when nothing else exists (the rules of
    include/photon/scheduler/inference_request.hpp:172-182)."""
    out = []
    while True:
        draw = uniform_draw(seed, len(out)) if temperature > 0 else 0.0
        out.append(token_after(list(prompt) + out, draw))
        if not ignore_eos and out[-1] == END:
            return out, "eos"
        if len(out) >= max_new:
            return out, "length"
        if len(prompt) + len(out) > max_model_len:
            return out, "max_model_len"


class _NoEvent:
    def record(self):
        pass

    def synchronize(self):
        pass


class StandInRunner:
    """ModelRunner's interface towards the engine and the scheduler, on the host."""

    graph_safe = True

    def __init__(self, options: EngineOptions, max_model_len: int, windows=(None,)):
        self.options = options
        self.max_model_len = max_model_len
        self.device = "cpu"
        self.workspace = None
        self.spec = types.SimpleNamespace(eos_token_ids=(END,), vocab_size=VOCAB)
        # one cache group per entry: all keys, or a window whose pages return while the request runs
        self.cache = CacheManager(list(windows), options.block_size, options.num_blocks, options.max_batch, max_model_len)
        self.history = {}            # rid -> the tokens in the cache, by position
        self._results = {}           # batch size -> the one buffer every step of that size writes
        self.decode_steps = self.mixed_steps = self.fed_steps = 0

    def admit(self, rid):
        slot = self.cache.admit(rid)
        self.history[rid] = []
        return slot

    def release(self, rid):
        self.cache.release(rid)
        del self.history[rid]

    def new_event(self):
        return _NoEvent()

    def host_token_buffer(self, n):
        return torch.empty(n, dtype=torch.int32)

    def _run(self, entries):
        seen = set()
        for e in entries:
            assert e.rid not in seen and e.rid in self.cache and len(e.tokens) > 0
            seen.add(e.rid)
            assert self.cache.length(e.rid) == len(self.history[e.rid])     # the step starts where the cache ends
            assert self.cache.length(e.rid) + len(e.tokens) <= self.max_model_len
        slots = [self.cache.slot(e.rid) for e in entries]
        self.cache.reserve_step(slots, [len(e.tokens) for e in entries])     # the whole step or OutOfPagesError
        wanted = []
        for e in entries:
            start = len(self.history[e.rid])
            self.history[e.rid].extend(int(t) for t in e.tokens)
            wanted += [tuple(self.history[e.rid][:start + w + 1]) for w in e.want]
        self.cache.commit_step(slots, [len(e.tokens) for e in entries])
        return wanted

    def step(self, entries):
        self.mixed_steps += 1
        return self._run(list(entries)) or None      # "logits": the histories, which StandInSampler turns into tokens

    def decode_step(self, entries, temperatures, uniforms, feed=None):
        entries = list(entries)
        assert all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)
        if feed is not None:
            ids, rows = feed
            assert len(rows) == len(entries)
            entries = [StepEntry(e.rid, [int(ids[r])], [0]) for e, r in zip(entries, rows)]
            self.fed_steps += 1
        self.decode_steps += 1
        wanted = self._run(entries)
        out = self._results.setdefault(len(entries), torch.zeros(len(entries), dtype=torch.int32))
        out.copy_(torch.tensor([token_after(h, u if t > 0 else 0.0) for h, t, u in zip(wanted, temperatures, uniforms)],
                               dtype=torch.int32))
        return out


class StandInSampler:
    def sample(self, logits, temperatures, uniforms):
        return [token_after(h, u if t > 0 else 0.0) for h, t, u in zip(logits, temperatures, uniforms)]


def make_engine(rng, lookahead, use_graphs, max_model_len=96):
    page = rng.choice([4, 8, 16])
    options = EngineOptions(block_size=page, num_blocks=rng.choice([6, 10, 16, 40, 200]), max_batch=rng.choice([1, 2, 3, 4, 6]),
                            max_step_tokens=rng.choice([4, 8, 16, 64]), chunk_size=rng.choice([2, 4, 8, 32]),
                            lookahead=lookahead, use_graphs=use_graphs, device="cpu")
    runner = StandInRunner(options, max_model_len, rng.choice([(None,), (None,), (None, 12), (20, None, 6)]))
    eng = ContinuousBatchEngine(None, runner=runner)
    eng.sampler = StandInSampler()
    return eng


def workload(rng, max_model_len, pool_tokens):
    reqs = []
    for _ in range(rng.randint(1, 10)):
        # every request alone must fit the pool, or the scheduler rightly ends it for want of pages
        longest = max(2, min(max_model_len - 2, pool_tokens - 2))
        n_prompt = rng.randint(1, min(40, longest - 1))
        max_new = rng.randint(1, 30)
        max_new = min(max_new, longest - n_prompt) if rng.random() < 0.8 else max_new
        reqs.append(dict(prompt=[rng.randrange(VOCAB) for _ in range(n_prompt)], max_new=max(1, max_new),
                         temperature=rng.choice([0.0, 0.0, 0.8]), seed=rng.randrange(1 << 30),
                         ignore_eos=rng.random() < 0.3, arrival=rng.randint(0, 25),
                         abort_at=rng.randint(0, 60) if rng.random() < 0.15 else None))
    return reqs


def drive(eng, reqs):
    order = sorted(range(len(reqs)), key=lambda i: reqs[i]["arrival"])
    ids, calls, aborted = {}, 0, {}          # aborted: request -> what it held when abort() returned
    while order or eng.has_work():
        while order and reqs[order[0]]["arrival"] <= calls:
            i = order.pop(0)
            r = reqs[i]
            ids[i] = eng.add_request(r["prompt"], r["max_new"], temperature=r["temperature"], seed=r["seed"],
                                     ignore_eos=r["ignore_eos"])
        for i, rid in ids.items():
            if reqs[i]["abort_at"] == calls and i not in aborted:
                if eng.abort(rid):
                    aborted[i] = list(eng.get_request(rid).generated_tokens)
        eng.step()
        eng.runner.cache.check_invariants()
        calls += 1
        assert calls < 20000, "the engine makes no progress"
    return ids, aborted


@pytest.mark.parametrize("lookahead,use_graphs", [(False, False), (False, True), (True, True)])
def test_random_workloads_give_every_request_its_own_tokens(lookahead, use_graphs):
    fed = preempted = ended_early = 0
    for seed in range(400):
        rng = random.Random(seed)
        max_model_len = rng.choice([48, 96])
        eng = make_engine(rng, lookahead, use_graphs, max_model_len)
        pool_tokens = eng.options.num_blocks * eng.options.block_size
        reqs = workload(rng, max_model_len, pool_tokens)
        ids, aborted = drive(eng, reqs)
        what = f"seed {seed} lookahead={lookahead} graphs={use_graphs}"
        for i, r in enumerate(reqs):
            req = eng.get_request(ids[i])
            want, reason = alone(r["prompt"], r["max_new"], r["temperature"], r["seed"], r["ignore_eos"], max_model_len)
            got = list(req.generated_tokens)
            if i in aborted:
                # what it had generated, and not a token more from a step that was still running
                assert req.finish_reason == "aborted" and got == aborted[i] == want[:len(got)], f"{what}: aborted request {i}"
                continue
            assert req.is_finished(), f"{what}: request {i} never finished"
            if req.finish_reason == "out_of_pages":      # a request that cannot fit the pool even alone
                needs = len(r["prompt"]) + len(got)
                assert needs + 1 > pool_tokens - eng.options.block_size and got == want[:len(got)], f"{what}: request {i} ended for want of pages"
                continue
            assert got == want and req.finish_reason == reason, f"{what}: request {i}: {got} != {want} ({req.finish_reason} / {reason})"
            ended_early += reason == "eos"
        assert eng.runner.cache.num_live == 0, what
        assert all(eng.runner.cache.free_pages(g) == eng.options.num_blocks for g in range(len(eng.runner.cache.groups))), what
        assert not eng.runner.history, what
        fed += eng.runner.fed_steps
        preempted += eng.get_stats().num_preemptions
    # the workloads did reach the paths they are for
    assert preempted > 20 and ended_early > 50
    assert (fed > 200) == lookahead


def test_a_step_ahead_reads_its_tokens_from_the_step_before():
    """All requests decoding and nobody waiting: every step but the first is launched from the
    device-side tokens of the one before, and the result is the same."""
    rng = random.Random(5)
    opts = EngineOptions(block_size=8, num_blocks=64, max_batch=4, max_step_tokens=64, chunk_size=32, lookahead=True, device="cpu")
    runner = StandInRunner(opts, 128)
    eng = ContinuousBatchEngine(None, runner=runner)
    eng.sampler = StandInSampler()
    prompts = [[rng.randrange(VOCAB) for _ in range(n)] for n in (5, 9, 3)]
    ids = [eng.add_request(p, 20, ignore_eos=True) for p in prompts]
    eng.run_until_complete()
    for rid, p in zip(ids, prompts):
        assert eng.get_result(rid) == alone(p, 20, 0.0, 0, True, 128)[0]
    assert runner.fed_steps >= 17 and runner.decode_steps == runner.fed_steps + 1


def test_engine_refuses_tokens_outside_the_vocabulary():
    opts = EngineOptions(block_size=8, num_blocks=8, max_batch=2, device="cpu")
    eng = ContinuousBatchEngine(None, runner=StandInRunner(opts, 64))
    with pytest.raises(RequestError):
        eng.add_request([1, VOCAB], 4)


def test_the_decision_to_copy_the_weights_for_streaming():
    """Left to itself a runner makes the copies only when they take at most half of the memory that
    is free after the weights; asked for by name they are made whenever they fit, and refused with
    the engine's own error when they do not."""
    from photon_infer_amd.engine.step import stream_copies_wanted
    from photon_infer_amd.errors import ErrorCode, OutOfMemoryError

    GiB = 1 << 30
    assert stream_copies_wanted(2 * GiB, 280 * GiB, asked=False)            # 1B sizes on an empty device
    assert stream_copies_wanted(16 * GiB, 250 * GiB, asked=False)           # 8B sizes
    assert not stream_copies_wanted(130 * GiB, 140 * GiB, asked=False)      # weights take half the device: none
    assert not stream_copies_wanted(71 * GiB, 140 * GiB, asked=False)
    assert stream_copies_wanted(70 * GiB, 140 * GiB, asked=False)
    assert not stream_copies_wanted(0, 140 * GiB, asked=False) and not stream_copies_wanted(0, 140 * GiB, asked=True)
    assert stream_copies_wanted(130 * GiB, 140 * GiB, asked=True)           # asked for: made while they fit
    with pytest.raises(OutOfMemoryError, match="stream_copies=True") as err:
        stream_copies_wanted(150 * GiB, 140 * GiB, asked=True)
    assert err.value.code == ErrorCode.OUT_OF_MEMORY


def test_kernels_launch_on_the_current_devices_stream(monkeypatch):
    """The stream handle that every kernel launch takes is asked for anew each time, for the
    device that is current then: a process may hold runners on several devices (a runner makes
    its own device current around its calls)."""
    from photon_infer_amd.ops import _lib

    current = {"device": 0}
    asked = []
    monkeypatch.setattr(_lib, "_CURRENT_DEVICE", lambda: current["device"])
    monkeypatch.setattr(_lib, "_RAW_STREAM", lambda index: asked.append(index) or 1000 + index)
    assert _lib.current_stream() == 1000
    current["device"] = 3
    assert _lib.current_stream() == 1003 and asked == [0, 3]
