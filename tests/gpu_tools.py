"""Helpers shared by the GPU tests."""
from __future__ import annotations

import io
import json
import os
from types import SimpleNamespace
from typing import Dict, List, Sequence

import numpy as np
import torch

DEV = "cuda:0"


def fp32_tol(ref: torch.Tensor) -> float:
    """float32 engine against the float32 plain implementation."""
    return 3e-5 * max(1.0, ref.abs().max().item())


def bf16_tol(ref: torch.Tensor, emulated: torch.Tensor) -> float:
    """bfloat16 engine against the float32 plain implementation.  The yardstick is what
    rounding activations to bfloat16 at the engine's rounding points does to the plain
    implementation itself (``emulated``): the engine may be off by three times the largest
    deviation that this rounding causes anywhere in the sequence, and no more."""
    return 3.0 * (emulated - ref).abs().max().item()


def tol_for(dtype: str, ref: torch.Tensor, emulated: torch.Tensor = None) -> float:
    return fp32_tol(ref) if dtype == "float32" else bf16_tol(ref, emulated)


class PagedKV:
    """Scatter dense per-request K/V [S, kv_heads, hd] into a page pool under a random page order."""

    def __init__(self, seqs: Sequence[tuple], page_size: int, dtype, seed: int = 0, spare_pages: int = 3):
        nkv, hd = seqs[0][0].shape[1:]
        blocks = [-(-k.shape[0] // page_size) for k, _ in seqs]
        total = sum(blocks) + spare_pages
        g = torch.Generator().manual_seed(seed)
        order = torch.randperm(total, generator=g).tolist()
        width = max(blocks)
        self.table = torch.full((len(seqs), width), -1, dtype=torch.int32)
        # unused pages hold large values: a read outside a request's keys shows
        self.k = torch.full((total, nkv, page_size, hd), 1e4, dtype=torch.float32)
        self.v = torch.full((total, nkv, hd, page_size), -1e4, dtype=torch.float32)   # values are kept transposed
        it = iter(order)
        for r, (k, v) in enumerate(seqs):
            for b in range(blocks[r]):
                page = next(it)
                self.table[r, b] = page
                n = min(page_size, k.shape[0] - b * page_size)
                self.k[page, :, :n] = k[b * page_size: b * page_size + n].transpose(0, 1)
                self.v[page, :, :, :n] = v[b * page_size: b * page_size + n].permute(1, 2, 0)
        self.k = self.k.to(dtype).to(DEV)
        self.v = self.v.to(dtype).to(DEV)
        self.table = self.table.to(DEV)
        self.page_size = page_size


def attention_ctx(q_lens: Sequence[int], kv_lens: Sequence[int], dtype) -> SimpleNamespace:
    """The fields of a StepContext that the attention kernels read, made as the step function makes them."""
    from photon_infer_amd import ops

    R = len(q_lens)
    q_start = np.zeros(R + 1, np.int32)
    np.cumsum(q_lens, out=q_start[1:])
    parts = {
        "positions": np.concatenate([np.arange(kv - n, kv, dtype=np.int32) for n, kv in zip(q_lens, kv_lens)]),
        "req_of_token": np.repeat(np.arange(R, dtype=np.int32), q_lens),
        "q_start": q_start, "kv_len": np.asarray(kv_lens, np.int32),
    }
    views = ops.upload_arrays(parts, DEV)
    # no runner here: no workspace (the ops take what they need per call) and no plans made
    # beforehand (the attention op makes its work list itself)
    return SimpleNamespace(T=int(sum(q_lens)), R=R, dtype=dtype, q_lens=list(q_lens), kv_lens=list(kv_lens),
                           max_q_len=max(q_lens), max_kv_len=max(kv_lens), all_decode=all(n == 1 for n in q_lens), scratch={},
                           workspace=None, plans={}, **{k: views[k] for k in ("positions", "req_of_token", "q_start", "kv_len")})


def run_trace(runner, steps: List[dict], out_dir: str) -> Dict[tuple, torch.Tensor]:
    """Replay ``steps`` through the framework's replay loop; {(id, position): logits row}."""
    from photon_infer_amd.engine.replay import replay

    lines = io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n")
    done = io.StringIO()
    replay(runner, lines, out_dir, done)
    assert done.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    return collect_logits(steps, out_dir, runner.spec.vocab_size)


def collect_logits(steps: List[dict], out_dir: str, vocab: int) -> Dict[tuple, torch.Tensor]:
    got, pos = {}, {}
    for s in steps:
        wanted = [(e["id"], pos.get(e["id"], 0) + w) for e in s["entries"] for w in e.get("want", [])]
        for e in s["entries"]:
            pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        for rid in s.get("end", []):
            pos.pop(rid, None)
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if not wanted:
            assert not os.path.exists(path)
            continue
        arr = np.fromfile(path, dtype="<f4").reshape(len(wanted), vocab)
        for key, row in zip(wanted, arr):
            assert key not in got
            got[key] = torch.from_numpy(row.copy())
    return got


def cut_steps(rid: str, tokens: Sequence[int], sizes: Sequence[int], first_step: int = 0, want_all: bool = True,
              end: bool = True) -> List[dict]:
    """Steps that feed ``tokens`` of one request in portions of ``sizes`` (cycled)."""
    steps, i, k = [], 0, 0
    while i < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - i)
        steps.append({"step": first_step + len(steps),
                      "entries": [{"id": rid, "tokens": list(tokens[i:i + n]), "want": list(range(n)) if want_all else []}],
                      "end": []})
        i += n
        k += 1
    if end:
        steps[-1]["end"] = [rid]
    return steps


def live_token_need(steps: List[dict], rounding: int = 64) -> int:
    """The --max-tokens a trace needs: most tokens live at once, each request rounded up."""
    held, worst = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // rounding) * rounding for n in held.values()))
        for rid in s.get("end", []):
            held.pop(rid, None)
    return worst
