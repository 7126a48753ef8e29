#!/usr/bin/python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode1b|long1b|serve3b|mixed8b]
                    [--batch 8,1,64] [--context 4096] [--dtype bf16|fp32]

Every workload prints ONE JSON line.  The default, ``decode1b`` (Llama 3.2 1B layer sizes):  ``value`` is decoded tokens per second at batch 8 with the context
length of the benchmark configuration (every request's cache holds that many tokens when
the timed steps end).  A "step" is one decode step of the whole batch through the engine's
own path, driven as the engine drives its decode phase: metadata upload, the replayed graph
(model + sampling kernel) that takes its tokens from the step before it on the device, and
the copy of the chosen tokens to the host, which reads every step's tokens one step late.
Also on the line: ``prefill`` (one 2,048-token prompt in one step), ``roofline`` (bytes the
decode step has to read / its time, against 8 TB/s) and ``points`` (batch 1 and 64, and
``decode_b8_fp32``: the headline's decode step on the float32 path).
``points`` also holds ``engine_b8``: decoded tokens per second of the same batch through
``ContinuousBatchEngine`` (scheduler, request objects, sampling, the step ahead), measured over its
decode phase.

``--batch a,b,c``: the first is the headline's batch, the others become ``points.decode_b<b>``;
``--context N``: the context length the decode steps end at.  ``--dtype fp32`` runs the same
workload on the float32 path (true 32-bit kernels; the caches are then filled with random
numbers instead of running 4,096-token prompts through them).

``--workload long1b`` (the same model): decode steps at further sizes over caches of random
numbers - batch 8 at a context of 32,768, one request at 131,000, batch 64 at 8,192 - and one
512-token portion of a prompt at the end of a context of 16,384, each with the bytes it has to
read or the flops it does against the peaks.  After demo/compare_batching_methods.cpp:251-309 of
the reference, which prints a throughput per workload.

``--workload serve3b`` (Llama 3.2 3B layer sizes): continuous batching of 64 requests, prompts of
128 to 2,048 tokens, 64 to 512 new tokens each, 16 there at the start and 4 more every 8 steps,
through ``ContinuousBatchEngine``: total tokens per second, preemptions, share of the time the host
waited for the GPU.  After demo/compare_batching_methods.cpp:251-309 of the reference.
``--workload mixed8b`` (Llama 3.1 8B layer sizes): steps that hold one 512-token portion of a
prompt late in a context of 8,192 beside 64 decoding requests at that context: milliseconds per
mixed step, and the step's flops and bytes against the peaks.

Weights are random (N(0, 0.02), norms 1), token ids uniform random; no dataset is involved.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# layer sizes of Llama 3.2 1B, the benchmark configuration
MODEL = dict(
    architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=8192, num_hidden_layers=16,
    num_attention_heads=32, num_key_value_heads=8, head_dim=64, vocab_size=128256,
    max_position_embeddings=131072, rms_norm_eps=1e-5, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True, torch_dtype="bfloat16",
)
# the other two benchmark configurations
MODEL_3B = dict(MODEL, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24, num_key_value_heads=8, head_dim=128,
                intermediate_size=8192)
MODEL_8B = dict(MODEL, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                intermediate_size=14336, tie_word_embeddings=False,
                rope_scaling=dict(MODEL["rope_scaling"], factor=8.0))
CONTEXT = 4096
PREFILL_TOKENS = 2048
BLOCK_SIZE = 16
HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def make_runner(cfg_raw, layers, dtype, max_batch, max_cache_tokens, seed=0, max_model_len=CONTEXT + 64, **options):
    import torch

    from photon_infer_amd.engine import EngineOptions, ModelRunner
    from photon_infer_amd.registry import build_model_spec, config_from_dict

    raw = dict(cfg_raw, num_hidden_layers=layers)
    cfg = config_from_dict(raw)
    spec = build_model_spec(cfg)
    tdtype = torch.bfloat16 if dtype == "bf16" else torch.float32
    gen = torch.Generator(device="cuda").manual_seed(seed)
    tensors = {}
    for s in spec.tensor_specs():
        if s.role == "norm":
            tensors[s.name] = torch.ones(s.shape, dtype=tdtype, device="cuda")
        else:
            tensors[s.name] = (torch.randn(s.shape, generator=gen, device="cuda", dtype=torch.float32) * 0.02).to(tdtype)
    opts = EngineOptions(dtype="bfloat16" if dtype == "bf16" else "float32", block_size=BLOCK_SIZE,
                         max_cache_tokens=max_cache_tokens, max_batch=max_batch, max_model_len=max_model_len, **options)
    return ModelRunner(None, opts, config=cfg, tensors=tensors), cfg


def weight_bytes(runner) -> int:
    """Bytes of every tensor the decode step reads once (tied head counted once)."""
    seen, total = set(), 0
    m = runner.model
    tensors = [m.head.weight, m.final_norm.weight]
    for b in m.blocks:
        tensors += [b.norm1.weight, b.norm2.weight, b.mixer.w_qkv, b.mixer.w_o, b.ffn.w_gate_up, b.ffn.w_down]
    for t in tensors:
        if t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()
    return total


def kv_bytes_per_token(cfg, layers, elem) -> int:
    return 2 * layers * cfg.num_key_value_heads * cfg.head_dim * elem


def prefill_flops(cfg, layers, T) -> float:
    per_layer = cfg.hidden_size * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * cfg.hidden_size \
        + 3 * cfg.hidden_size * cfg.intermediate_size
    gemm = 2.0 * T * per_layer * layers
    attn = layers * 2 * 2.0 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2)
    head = 2.0 * cfg.hidden_size * cfg.vocab_size
    return gemm + attn + head


def time_decode(runner, batch, steps, warmup, context, seed=1, synthetic_cache=False):
    """Plain timing of ``steps`` decode steps of ``batch`` requests that end at ``context``.
    ``synthetic_cache``: instead of running the prompts through the model, reserve the pages
    and fill the pools with random numbers (for profiles that should hold decode kernels only)."""
    import torch

    from photon_infer_amd.engine import StepEntry

    vocab = runner.spec.vocab_size
    g = torch.Generator().manual_seed(seed)
    start_len = context - steps - warmup
    assert start_len >= 1
    rids = [f"d{batch}_{i}" for i in range(batch)]
    for rid in rids:
        runner.admit(rid)
        if synthetic_cache:
            runner.cache.reserve(rid, start_len)
            runner.cache.commit(rid, start_len)
            continue
        toks = torch.randint(0, vocab, (start_len,), generator=g).tolist()
        for i in range(0, start_len, 2048):
            runner.step([StepEntry(rid, toks[i:i + 2048])])
    if synthetic_cache:
        for lc in runner.layer_caches:
            lc.k.normal_()
            lc.v.normal_()
    last = torch.randint(0, vocab, (batch,), generator=g).tolist()
    temps, draws = [0.0] * batch, [0.0] * batch
    rows = list(range(batch))
    host = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)]
    arrived = [torch.cuda.Event(), torch.cuda.Event()]

    # The loop of the engine's decode phase: a step takes its tokens from the step before it on
    # the device, and the host reads a step's tokens while the next one runs (one step late).
    def run(n, ids):
        for i in range(n):
            if ids is None:
                ids = runner.decode_step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, last)], temps, draws)
            else:
                ids = runner.decode_step([StepEntry(rid, [0], [0]) for rid in rids], temps, draws, (ids, rows))
            host[i % 2].copy_(ids, non_blocking=True)
            arrived[i % 2].record()
            if i:
                arrived[(i - 1) % 2].synchronize()
                host[(i - 1) % 2].tolist()
        return ids

    ids = run(warmup, None)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(steps, ids)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    mean_ctx = context - (steps - 1) / 2.0        # keys each request reads, averaged over the timed steps
    for rid in rids:
        runner.release(rid)
    return dt / steps, mean_ctx


def time_prefill(runner, tokens, reps, seed=2):
    import torch

    from photon_infer_amd.engine import StepEntry

    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(0, runner.spec.vocab_size, (tokens,), generator=g).tolist()

    def once(i):
        rid = f"p{i}"
        runner.admit(rid)
        logits = runner.step([StepEntry(rid, toks, [tokens - 1])])
        runner.release(rid)
        return logits

    once(-1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(reps):
        once(i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def time_engine_decode(runner, batch, steps, warmup, context, seed=3):
    """Seconds per decode step of ``batch`` requests through ContinuousBatchEngine with its default
    options: the prompts run first (untimed, with ``warmup`` decode steps), then ``steps`` engine
    steps are timed while every request decodes."""
    import torch

    from photon_infer_amd import ContinuousBatchEngine

    eng = ContinuousBatchEngine(None, runner=runner)
    g = torch.Generator().manual_seed(seed)
    prompt_len = context - steps - warmup - 2
    for _ in range(batch):
        eng.add_request(torch.randint(0, runner.spec.vocab_size, (prompt_len,), generator=g).tolist(),
                        steps + warmup + 2, ignore_eos=True)
    reqs = list(eng.scheduler.requests.values())
    while min(r.num_generated() for r in reqs) < warmup:
        eng.step()
    torch.cuda.synchronize()
    n0, t0 = eng.steps, time.perf_counter()
    while eng.steps - n0 < steps and eng.has_work():
        eng.step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / max(1, eng.steps - n0)
    eng.run_until_complete()
    return sec


def workload_serve3b(args) -> int:
    """Continuous batching at Llama 3.2 3B layer sizes (see the module text)."""
    import collections
    import random

    import torch

    from photon_infer_amd import ContinuousBatchEngine

    layers = args.layers or MODEL_3B["num_hidden_layers"]
    n_req, first, more, every = 64, 16, 4, 8
    rng = random.Random(0)
    shapes = [(rng.randint(128, 2048), rng.randint(64, 512)) for _ in range(n_req)]
    cache_tokens = n_req * 2624            # every request at its longest, to the page
    runner, cfg = make_runner(MODEL_3B, layers, args.dtype, n_req, cache_tokens, max_model_len=2048 + 512 + 64,
                              max_step_tokens=2048, chunk_size=512)

    def run():
        eng = ContinuousBatchEngine(None, runner=runner)
        g = torch.Generator().manual_seed(0)
        pending = collections.deque(shapes)

        def admit(n):
            for _ in range(min(n, len(pending))):
                p, o = pending.popleft()
                eng.add_request(torch.randint(0, cfg.vocab_size, (p,), generator=g).tolist(), o, ignore_eos=True)

        admit(first)
        torch.cuda.synchronize()
        t0, calls = time.perf_counter(), 0
        while eng.has_work() or pending:
            eng.step()
            calls += 1
            if calls % every == 0:
                admit(more)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, eng

    run()                                   # untimed: captures the decode graphs of every batch size it meets
    sec, eng = run()
    reqs = list(eng.scheduler.requests.values())
    generated = sum(r.num_generated() for r in reqs)
    prompt = sum(p for p, _ in shapes)
    assert generated == sum(o for _, o in shapes) and all(r.finish_reason == "length" for r in reqs)
    stats = eng.get_stats()
    elem = 2 if args.dtype == "bf16" else 4
    line = {
        "metric": "total tok/s (prompt + generated), continuous batching of 64 requests (Llama 3.2 3B layer sizes, random weights)",
        "value": round((prompt + generated) / sec, 1), "unit": "tokens/s", "n_gpus": 1, "steps": eng.steps, "warmup": 0,
        "ms_per_step": round(sec / eng.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
        "config": {
            "model": "llama-3.2-3b-sizes", "layers": layers, "layers_of_model": MODEL_3B["num_hidden_layers"],
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "tied_embeddings": cfg.tie_word_embeddings, "requests": n_req, "prompt_lengths": "uniform 128..2048",
            "output_lengths": "uniform 64..512", "admission": f"{first} at the start, {more} every {every} steps",
            "chunk_size": 512, "max_step_tokens": 2048, "kv_block": BLOCK_SIZE, "cache_tokens": cache_tokens,
            "parallelism": "single-gpu",
        },
        "seconds": round(sec, 3), "prompt_tokens": prompt, "generated_tokens": generated,
        "generated_tok_per_s": round(generated / sec, 1), "preemptions": stats.num_preemptions,
        "host_wait_share": round(eng.host_wait_seconds / sec, 3), "graphs": len(runner._graphs),
        "weight_bytes": weight_bytes(runner), "kv_bytes_per_token": kv_bytes_per_token(cfg, layers, elem),
    }
    print(json.dumps(line), flush=True)
    return 0


def time_late_portion(runner, portion, context, reps, seed=4):
    """Seconds per step of one ``portion``-token piece of a prompt that ends at ``context``, over
    a cache of random numbers (the pages before it reserved, not computed)."""
    import torch

    from photon_infer_amd.engine import StepEntry

    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(0, runner.spec.vocab_size, (portion,), generator=g).tolist()

    def once(i):
        rid = f"late{i}"
        runner.admit(rid)
        runner.cache.reserve(rid, context - portion)
        runner.cache.commit(rid, context - portion)
        runner.step([StepEntry(rid, toks, [portion - 1])])
        runner.release(rid)

    once(-1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(reps):
        once(i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def workload_long1b(args) -> int:
    """Decode steps and a late prompt portion at long contexts, Llama 3.2 1B layer sizes (see the
    module text).  One runner whose pool holds the largest case."""
    layers = args.layers or MODEL["num_hidden_layers"]
    cases = [(8, 32768), (1, 131000), (64, 8192)]
    portion, portion_ctx = 512, 16384
    pool = max(b * (c + 64) for b, c in cases)
    runner, cfg = make_runner(MODEL, layers, args.dtype, 64, pool, max_model_len=131072)
    elem = 2 if args.dtype == "bf16" else 4
    wbytes, kvb = weight_bytes(runner), kv_bytes_per_token(cfg, layers, elem)
    points = {}
    for b, c in cases:
        sec, mean_ctx = time_decode(runner, b, args.steps, args.warmup, c, synthetic_cache=True)
        gbs = (wbytes + b * mean_ctx * kvb) / sec / 1e9
        points[f"decode_b{b}_ctx{c}"] = {"ms_per_step": round(sec * 1e3, 4), "tokens_per_s": round(b / sec, 1),
                                         "GB_per_s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    psec = time_late_portion(runner, portion, portion_ctx, max(2, min(8, args.steps)))
    per_layer = cfg.hidden_size * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * cfg.hidden_size + 3 * cfg.hidden_size * cfg.intermediate_size
    flops = 2.0 * portion * per_layer * layers + 2.0 * cfg.hidden_size * cfg.vocab_size \
        + layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * portion * (portion_ctx - portion / 2.0)
    points[f"portion{portion}_ctx{portion_ctx}"] = {"ms": round(psec * 1e3, 3), "tokens_per_s": round(portion / psec, 1),
                                                    "frac_of_flops_peak": round(flops / psec / PEAK_FLOPS[args.dtype], 4)}
    head = points["decode_b8_ctx32768"]
    line = {
        "metric": "decode tok/s at batch 8, context 32768 (Llama 3.2 1B layer sizes, random weights, random cache contents)",
        "value": head["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), random cache contents, uniform random token ids",
        "config": {
            "model": "llama-3.2-1b-sizes", "layers": layers, "layers_of_model": MODEL["num_hidden_layers"],
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "tied_embeddings": cfg.tie_word_embeddings, "global_batch": 8, "seq_len": 32768, "kv_block": BLOCK_SIZE,
            "parallelism": "single-gpu", "weight_bytes": wbytes, "kv_bytes_per_token": kvb,
        },
        "roofline": {"bound": "hbm", "achieved": head["GB_per_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["frac_of_hbm_peak"]},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


def workload_mixed8b(args) -> int:
    """Mixed steps at Llama 3.1 8B layer sizes (see the module text)."""
    import torch

    from photon_infer_amd.engine import StepEntry

    layers = args.layers or MODEL_8B["num_hidden_layers"]
    ctx, portion, ndec = 8192, 512, 64
    reps = max(2, min(4, args.steps))        # the timed portions cover the last 2,048 tokens of the context
    runner, cfg = make_runner(MODEL_8B, layers, args.dtype, ndec + 1, (ndec + 1) * (ctx + 64), max_model_len=ctx + 64)
    elem = 2 if args.dtype == "bf16" else 4
    first = ctx - portion * (reps + 1)       # the portions that are timed end at ctx
    rids = [f"d{i}" for i in range(ndec)]
    for rid in rids:                         # the decoding requests: pages reserved, contents random
        runner.admit(rid)
        runner.cache.reserve(rid, ctx - reps - 2)
        runner.cache.commit(rid, ctx - reps - 2)
    runner.admit("p")
    runner.cache.reserve("p", first)
    runner.cache.commit("p", first)
    for lc in runner.layer_caches:
        lc.k.normal_()
        lc.v.normal_()
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, cfg.vocab_size, (ctx,), generator=g).tolist()
    state = {"pos": first}

    def mixed():
        p = state["pos"]
        runner.step([StepEntry("p", prompt[p:p + portion], [])] + [StepEntry(r, [5], [0]) for r in rids])
        state["pos"] = p + portion

    mixed()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        mixed()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / reps
    tokens = portion + ndec
    mean_ctx = ctx - portion * (reps - 1) / 2.0 - portion / 2.0       # keys a portion's token sees, averaged over the timed steps
    per_layer = cfg.hidden_size * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * cfg.hidden_size + 3 * cfg.hidden_size * cfg.intermediate_size
    flops = 2.0 * tokens * per_layer * layers + 2.0 * ndec * cfg.hidden_size * cfg.vocab_size \
        + layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * (portion * mean_ctx + ndec * ctx)
    kvb = kv_bytes_per_token(cfg, layers, elem)
    step_bytes = weight_bytes(runner) + (ndec * ctx + mean_ctx + portion / 2.0) * kvb
    line = {
        "metric": "ms per mixed step: one 512-token prompt portion late in a context of 8192 beside 64 decoding requests (Llama 3.1 8B layer sizes, random weights)",
        "value": round(sec * 1e3, 3), "unit": "ms", "n_gpus": 1, "steps": reps, "warmup": 1, "ms_per_step": round(sec * 1e3, 3),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), random cache contents, uniform random token ids",
        "config": {
            "model": "llama-3.1-8b-sizes", "layers": layers, "layers_of_model": MODEL_8B["num_hidden_layers"],
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "tied_embeddings": cfg.tie_word_embeddings, "context": ctx, "portion_tokens": portion, "decoding_requests": ndec,
            "kv_block": BLOCK_SIZE, "parallelism": "single-gpu",
        },
        "tokens_per_s": round(tokens / sec, 1),
        "compute": {"flops": flops, "achieved": round(flops / sec / 1e12, 1), "peak": PEAK_FLOPS[args.dtype] / 1e12, "unit": "TFLOP/s",
                    "frac": round(flops / sec / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(step_bytes / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(step_bytes / sec / 1e9 / HBM_PEAK_GBS, 4)},
    }
    print(json.dumps(line), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", default="8,1,64",
                    help="batch sizes of the decode steps: the first is the headline's, the others become points")
    ap.add_argument("--context", type=int, default=CONTEXT, help="context length that the decode steps end at")
    ap.add_argument("--workload", choices=["decode1b", "long1b", "serve3b", "mixed8b"], default="decode1b")
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the model has, if memory or time needs it (both numbers are reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--only", choices=["decode", "prefill"], default=None,
                    help="run just the decode steps at --batch, or just the prefill (for profiling); prints a short line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU available", file=sys.stderr)
        return 1
    batches = [int(b) for b in str(args.batch).split(",") if b]
    if not batches or min(batches) < 1:
        print(f"bench.py: --batch {args.batch} names no batch size", file=sys.stderr)
        return 1
    args.batch, more_batches = batches[0], batches[1:]
    context = args.context
    if context <= args.steps + args.warmup:
        print(f"bench.py: --context {context} is shorter than the {args.steps + args.warmup} steps to run", file=sys.stderr)
        return 1
    if args.workload == "long1b":
        return workload_long1b(args)
    if args.workload == "serve3b":
        return workload_serve3b(args)
    if args.workload == "mixed8b":
        return workload_mixed8b(args)
    args.layers = args.layers or MODEL["num_hidden_layers"]
    elem = 2 if args.dtype == "bf16" else 4
    big = args.batch if (args.no_points or args.only) else max(batches)
    synthetic = args.dtype == "fp32"      # the float32 kernels would spend minutes on the prompts that fill the caches
    runner, cfg = make_runner(MODEL, args.layers, args.dtype, big, max(big * (context + 64), PREFILL_TOKENS + 64),
                              max_model_len=max(context, PREFILL_TOKENS) + 64)
    wbytes = weight_bytes(runner)
    kvb = kv_bytes_per_token(cfg, args.layers, elem)
    if args.only == "prefill":
        psec = time_prefill(runner, PREFILL_TOKENS, max(1, args.steps // 8))
        print(json.dumps({"only": "prefill", "tokens": PREFILL_TOKENS, "ms": round(psec * 1e3, 3)}), flush=True)
        return 0
    if args.only == "decode":
        sec, _ = time_decode(runner, args.batch, args.steps, args.warmup, context, synthetic_cache=True)
        print(json.dumps({"only": "decode", "batch": args.batch, "ms_per_step": round(sec * 1e3, 4),
                          "cache": "random numbers, no prompt was run"}), flush=True)
        return 0

    sec, mean_ctx = time_decode(runner, args.batch, args.steps, args.warmup, context, synthetic_cache=synthetic)
    value = args.batch / sec
    step_bytes = wbytes + args.batch * mean_ctx * kvb
    achieved = step_bytes / sec / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch}, context {context} (Llama 3.2 1B layer sizes, random weights)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), uniform random token ids"
                + (", random cache contents" if synthetic else ""),
        "config": {
            "model": "llama-3.2-1b-sizes", "layers": args.layers, "layers_of_model": MODEL["num_hidden_layers"],
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "tied_embeddings": cfg.tie_word_embeddings, "rope": "llama3 theta=500000 factor=32",
            "global_batch": args.batch, "seq_len": context, "kv_block": BLOCK_SIZE, "prefill_tokens": PREFILL_TOKENS,
            "parallelism": "single-gpu", "weight_bytes": wbytes, "kv_bytes_per_token": kvb,
            "weight_copies_in_streaming_order": runner.stream_copies,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        psec = time_prefill(runner, PREFILL_TOKENS, 5)
        flops = prefill_flops(cfg, args.layers, PREFILL_TOKENS)
        line["prefill"] = {"value": round(PREFILL_TOKENS / psec, 1), "tokens": PREFILL_TOKENS, "ms": round(psec * 1e3, 3),
                           "frac": round(flops / psec / PEAK_FLOPS[args.dtype], 4)}
        points = {}
        for b in more_batches:
            s, _ = time_decode(runner, b, args.steps, args.warmup, context, synthetic_cache=synthetic)
            points[f"decode_b{b}"] = round(b / s, 1)
        if not synthetic:
            points[f"engine_b{args.batch}"] = round(
                args.batch / time_engine_decode(runner, args.batch, args.steps, args.warmup, context), 1)
        if args.dtype == "bf16":
            # the same decode step on the float32 path (true 32-bit kernels, caches of random numbers)
            import gc
            del runner
            gc.collect()
            torch.cuda.empty_cache()
            runner32, _ = make_runner(MODEL, args.layers, "fp32", args.batch, args.batch * (context + 64), max_model_len=context + 64)
            s32, _ = time_decode(runner32, args.batch, min(args.steps, 16), min(args.warmup, 2), context, synthetic_cache=True)
            points[f"decode_b{args.batch}_fp32"] = round(args.batch / s32, 1)
        line["points"] = points
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
