"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled.  The replay drives the same ``ModelRunner.step`` (model, cache
manager, kernels) that generation uses; it owns no forward pass, cache or loader.

Input, one JSON object per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

A request is admitted when first seen and released when a step's ``end`` names it.  For
a step with wanted rows, ``<out>/<step>.f32`` holds the float32 logits [wanted, vocab] in
the order of the entries and of each ``want``.  After every step ``done <step>`` is
printed and flushed.
"""
from __future__ import annotations

import json
import os
import shutil
import sys
from typing import IO, Optional

import numpy as np

from ..errors import PhotonError
from .options import EngineOptions
from .step import ModelRunner, StepEntry

MAX_LIVE_REQUESTS = 8        # a trace holds up to four; some room to spare
TOKEN_ROUNDING = 64          # --max-tokens counts each request rounded up to this


def make_runner(model_dir: str, dtype: str, max_tokens: int, block_size: int = 16) -> ModelRunner:
    """A runner whose page pool holds exactly ``max_tokens`` tokens."""
    if TOKEN_ROUNDING % block_size:
        raise PhotonError(f"block size {block_size} must divide {TOKEN_ROUNDING}")
    options = EngineOptions(dtype=dtype, block_size=block_size, num_blocks=max(1, -(-max_tokens // block_size)),
                            max_batch=MAX_LIVE_REQUESTS, use_graphs=False)
    return ModelRunner(model_dir, options)


def replay(runner: ModelRunner, lines: IO[str], out_dir: str, done: Optional[IO[str]] = None) -> int:
    """Run every step read from ``lines``; returns the number of steps run."""
    os.makedirs(out_dir, exist_ok=True)
    steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step_id = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in runner.cache:
                runner.admit(rid)
            entries.append(StepEntry(rid, [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        logits = runner.step(entries)
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(out_dir, f".{step_id}.f32.tmp")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{step_id}.f32"))
        for rid in rec.get("end", []):
            if rid in runner.cache:
                runner.release(rid)
        steps += 1
        if done is not None:
            done.write(f"done {step_id}\n")
            done.flush()
    return steps


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(prog="trace_run", description="Replay a token trace and dump logits.")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each rounded up to a multiple of 64")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page (divides 64)")
    ap.add_argument("--random-weights", action="store_true",
                    help="--model names a bare config.json (or a folder that holds only one); weights are drawn from --seed")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--weight-std", type=float, default=0.02)
    args = ap.parse_args(argv)
    scratch = None
    try:
        model = args.model
        if args.random_weights:
            from ..weights import random_model_folder
            model = scratch = random_model_folder(args.model, seed=args.seed, std=args.weight_std)
        runner = make_runner(model, args.dtype, args.max_tokens, args.block_size)
        if scratch is not None:       # the weights are on the device now
            shutil.rmtree(scratch, ignore_errors=True)
            scratch = None
        replay(runner, sys.stdin, args.out, sys.stdout)
    except PhotonError as e:
        print(f"trace_run: {e}", file=sys.stderr, flush=True)
        return 1
    finally:
        if scratch is not None:
            shutil.rmtree(scratch, ignore_errors=True)
    return 0
