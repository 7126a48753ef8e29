"""Trace replay against the plain implementation, in float32 and in bfloat16:
whole requests; most in one step and the last 32 tokens one by one; portions of changing
size down to two tokens; up to four live requests mixed with so few pages that they are
used again; long decoding; the first tokens of a sequence; and the command itself."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
from gpu_tools import collect_logits, cut_steps, live_token_need, run_trace, tol_for
from tiny_models import ALL, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
MODELS = ["A", "B", "C", "D", "E", "F", "G", "H"]

_plain_cache = {}


def plain_logits(model_dir, tokens, emulate_bf16=False):
    key = (model_dir, tuple(tokens), emulate_bf16)
    if key not in _plain_cache:
        cfg, W = P.read_model_folder(model_dir)
        _plain_cache[key] = P.llama_forward(cfg, W, list(tokens), act_round=P.bf16_round if emulate_bf16 else None)
    return _plain_cache[key]


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_model_dir(root, name, seed=11) for name in MODELS}


def runner_for(model_dir, name, dtype, max_tokens):
    from photon_infer_amd.engine.replay import make_runner
    return make_runner(model_dir, dtype, max_tokens, ALL[name][1]["block_size"])


def requests_for(name, lengths, seed=0):
    vocab = ALL[name][0]["vocab_size"]
    return {f"r{i}": random_tokens(n, vocab, seed * 100 + i) for i, n in enumerate(lengths)}


def check(got, model_dir, reqs, dtype, what):
    assert got, "no logits came back"
    worst = 0.0
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, toks)
        tol = tol_for(dtype, ref, plain_logits(model_dir, toks, True) if dtype == "bfloat16" else None)
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: logits of {rid} position {p} are missing"
            err = (got[(rid, p)] - ref[p]).abs().max().item()
            worst = max(worst, err / tol)
            assert err <= tol, f"{what}: {rid} position {p}: error {err:.3e} > {tol:.3e} (first wrong position)"
    return worst


LENGTHS = {"A": [5, 9, 17, 70, 128], "B": [1, 7, 33, 64, 100, 200], "C": [3, 48, 131], "D": [1, 31, 65, 300], "E": [2, 33, 129, 260],
           "F": [1, 140, 300], "G": [2, 50, 270], "H": [3, 70, 260]}


def check_kernel_selection(runner, name, dtype, decoded_alone=False):
    """Model F is there so that the kernels chosen at real sizes run inside these comparisons: in
    bfloat16 its o and down projections are split over k and left in pieces that the next norm
    adds, and its q|k|v projection reaches the rotation (portions) or the fused decode kernel
    (single tokens) in pieces; where steps of single tokens alone ran late in a sequence
    (``decoded_alone``), attention left its key ranges for the o projection to merge.  The
    workspace counts say whether a run went that way."""
    counts = runner.workspace.counts
    if name != "F" or dtype != "bfloat16":
        if dtype == "float32":
            assert not counts, counts                   # the general kernels split nothing
        return
    assert counts["split_products"] > 0 and counts["deferred"] > 0 and counts["qkv_pieces"] > 0, counts
    assert counts["added_by_norm"] == counts["deferred"] - counts["flushed"] - counts["applied"] - counts["discarded"], counts
    assert counts["flushed"] == 0, counts               # every pending update found its norm
    if decoded_alone:
        assert counts["ranges_merged_by_product"] > 0, counts


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_each_request_alone_and_whole(model_dirs, tmp_path, name, dtype):
    reqs = requests_for(name, LENGTHS[name])
    steps = []
    for rid, toks in reqs.items():
        steps += cut_steps(rid, toks, [len(toks)], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    got = run_trace(runner, steps, str(tmp_path))
    check(got, model_dirs[name], reqs, dtype, "whole")
    check_kernel_selection(runner, name, dtype)
    assert runner.cache.num_live == 0 and runner.cache.free_pages() == runner.num_pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_last_32_tokens_one_by_one(model_dirs, tmp_path, name, dtype):
    n = {"A": 100, "B": 180, "C": 150, "D": 260, "E": 200, "F": 290, "G": 190, "H": 210}[name]
    reqs = requests_for(name, [n], seed=1)
    toks = reqs["r0"]
    steps = cut_steps("r0", toks, [n - 32] + [1] * 32)
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, "tail decoded")
    check_kernel_selection(runner, name, dtype, decoded_alone=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_portions_of_changing_size(model_dirs, tmp_path, name, dtype):
    n = {"A": 120, "B": 230, "C": 170, "D": 290, "E": 210, "F": 280, "G": 200, "H": 220}[name]
    reqs = requests_for(name, [n], seed=2)
    # F also in portions that the tile kernels take (more than 128 tokens), split over k
    for sizes in ([7, 2, 16, 3, 2, 33, 1, 5], [2], [64, 2, 2, 19]) + (([130, 2, 140],) if name == "F" else ()):
        steps = cut_steps("r0", reqs["r0"], sizes)
        runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
        check(run_trace(runner, steps, str(tmp_path / f"s{sizes[0]}_{len(sizes)}")), model_dirs[name], reqs, dtype,
              f"portions {sizes}")
        check_kernel_selection(runner, name, dtype)


def mixed_trace(reqs, patterns, max_live=4):
    """Up to ``max_live`` requests at a time; each live request brings its next portion (sizes
    from its pattern, so portions of some sit beside single tokens of others); a request
    that is through ends and the next one starts in the following step."""
    waiting = list(reqs)
    live, done_at, steps = [], {}, []
    fed = {rid: 0 for rid in reqs}
    turn = {rid: 0 for rid in reqs}
    index = {rid: i for i, rid in enumerate(reqs)}
    tick = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            live.append(waiting.pop(0))
        entries, ended = [], []
        tick += 1
        for rid in list(live):
            if (tick + index[rid]) % 5 == 4 and len(live) > 1:
                continue                                       # sits this step out, goes on later
            pat = patterns[rid]
            n = min(pat[turn[rid] % len(pat)], len(reqs[rid]) - fed[rid])
            turn[rid] += 1
            entries.append({"id": rid, "tokens": reqs[rid][fed[rid]:fed[rid] + n], "want": list(range(n))})
            fed[rid] += n
            if fed[rid] == len(reqs[rid]):
                ended.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_mixed_requests_with_pages_used_again(model_dirs, tmp_path, name, dtype):
    lengths = {"A": [40, 9, 128, 77, 5, 100, 64, 30], "B": [100, 1, 33, 250, 64, 7, 180, 90],
               "C": [131, 48, 3, 200, 96, 150], "D": [300, 65, 2, 129, 500, 17, 210],
               "E": [260, 33, 2, 129, 400, 64, 97], "F": [300, 65, 2, 129, 260, 17, 210],
               "G": [200, 33, 2, 129, 300, 64, 80], "H": [180, 33, 2, 129, 290, 64, 70]}[name]
    reqs = requests_for(name, lengths, seed=3)
    pats = [[16, 1, 1, 1, 2], [1], [33, 2, 7], [64, 1, 1], [5, 3, 2], [2, 2, 50], [1, 1, 1, 40], [9]]
    patterns = {rid: pats[i % len(pats)] for i, rid in enumerate(reqs)}
    steps = mixed_trace(reqs, patterns)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len({len(e["tokens"]) == 1 for e in s["entries"]}) == 2 for s in steps)   # portions beside single tokens
    need = live_token_need(steps)
    assert need < sum(-(-n // 64) * 64 for n in lengths)       # the pool cannot hold them all: pages come back
    runner = runner_for(model_dirs[name], name, dtype, need)
    owners = {}                                                # page -> requests that held it
    orig_reserve = runner.cache.reserve_step

    def spy(slots, tokens):
        orig_reserve(slots, tokens)
        for rid in list(reqs):
            if rid in runner.cache and runner.cache.slot(rid) in slots:
                for p in runner.cache.table_rows(0, [runner.cache.slot(rid)])[0]:
                    if p >= 0:
                        owners.setdefault(int(p), set()).add(rid)
    runner.cache.reserve_step = spy
    got = run_trace(runner, steps, str(tmp_path))
    assert any(len(v) > 1 for v in owners.values()), "no page was handed out a second time"
    check(got, model_dirs[name], reqs, dtype, "mixed")
    check_kernel_selection(runner, name, dtype)
    runner.cache.check_invariants()
    assert runner.cache.num_live == 0 and runner.cache.free_pages() == runner.num_pages


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(model_dirs, tmp_path, dtype):
    reqs = requests_for("B", [256], seed=4)            # to the model's last position
    steps = cut_steps("r0", reqs["r0"], [6] + [1] * 250)
    runner = runner_for(model_dirs["B"], "B", dtype, 256)
    check(run_trace(runner, steps, str(tmp_path)), model_dirs["B"], reqs, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_late_portions_of_a_long_prompt(model_dirs, tmp_path, dtype, monkeypatch):
    """Short portions near the end of the longest context the model allows, beside a second
    request's single tokens: in bfloat16 the portions' few tiles have their key ranges cut
    into shares, and the single tokens go to the key-split kernel in the same step."""
    reqs = requests_for("D", [1500, 130], seed=6)
    a = cut_steps("r0", reqs["r0"], [1440, 40, 3, 17])
    b = cut_steps("r1", reqs["r1"], [127, 1, 1, 1])
    steps = [b[0], a[0]]
    for i in range(1, 4):                                   # steps that hold a late portion of r0 and one token of r1
        steps.append({"entries": a[i]["entries"] + b[i]["entries"], "end": a[i]["end"] + b[i]["end"]})
    for i, st in enumerate(steps):
        st["step"] = i
    from photon_infer_amd.ops import fast
    cuts_made, count = [], fast.cut_count
    monkeypatch.setattr(fast, "cut_count", lambda walks, seats: cuts_made.append(count(walks, seats)) or cuts_made[-1])
    runner = runner_for(model_dirs["D"], "D", dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs["D"], reqs, dtype, "late portions")
    if dtype == "bfloat16":
        assert max(cuts_made) > 1, "no tile's key range was cut: the test does not reach what it is for"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_first_tokens_of_a_sequence(model_dirs, tmp_path, name, dtype):
    reqs = requests_for(name, [4, 4, 4], seed=5)
    steps = cut_steps("r0", reqs["r0"], [1, 1, 1, 1]) + cut_steps("r1", reqs["r1"], [2, 2], first_step=4) \
        + cut_steps("r2", reqs["r2"], [1, 3], first_step=6)
    runner = runner_for(model_dirs[name], name, dtype, 64)
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, "first tokens")


def test_step_preconditions(model_dirs):
    from photon_infer_amd import CacheError, OutOfPagesError, RequestError
    from photon_infer_amd.engine import StepEntry
    runner = runner_for(model_dirs["A"], "A", "float32", 64)
    with pytest.raises(CacheError, match="not live"):
        runner.step([StepEntry("x", [1, 2])])
    runner.admit("x")
    with pytest.raises(RequestError, match="vocabulary"):
        runner.step([StepEntry("x", [1, 256])])
    with pytest.raises(RequestError, match="no tokens"):
        runner.step([StepEntry("x", [])])
    with pytest.raises(RequestError, match="twice"):
        runner.step([StepEntry("x", [1]), StepEntry("x", [2])])
    with pytest.raises(RequestError, match="wanted row"):
        runner.step([StepEntry("x", [1, 2], [2])])
    with pytest.raises(RequestError, match="wanted twice"):
        runner.step([StepEntry("x", [1, 2], [0, 1, 0])])
    runner.admit("y")
    with pytest.raises(OutOfPagesError):
        runner.step([StepEntry("x", [1] * 40), StepEntry("y", [1] * 40)])
    assert runner.cache.free_pages() == runner.num_pages            # the refused step took nothing
    assert runner.step([StepEntry("x", [1] * 40)]) is None          # nothing wanted
    with pytest.raises(RequestError, match="limit"):
        runner.step([StepEntry("x", [1] * 100)])


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_command_itself(model_dirs, tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON lines in, 'done <step>' lines and .f32 files out."""
    reqs = requests_for("B", [70, 33], seed=6)
    steps = mixed_trace(reqs, {"r0": [16, 1, 2], "r1": [1, 5]})
    out = tmp_path / "out"
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", model_dirs["B"], "--dtype", dtype, "--out", str(out),
         "--max-tokens", str(live_token_need(steps))],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    got = collect_logits(steps, str(out), ALL["B"][0]["vocab_size"])
    check(got, model_dirs["B"], reqs, dtype, "command")


def test_the_command_from_a_bare_configuration_and_a_seed(tmp_path):
    """--random-weights: the model is a config.json alone; the weights are those that the
    random-weights mode writes for that configuration and seed."""
    from photon_infer_amd.config import LlamaConfig
    from photon_infer_amd.weights import write_random_model

    (tmp_path / "bare").mkdir()
    (tmp_path / "bare" / "config.json").write_text(json.dumps(ALL["B"][0]))
    written = write_random_model(LlamaConfig.from_dict(ALL["B"][0]), str(tmp_path / "written"), seed=9, std=0.05)
    reqs = requests_for("B", [41, 18], seed=8)
    steps = mixed_trace(reqs, {"r0": [16, 3], "r1": [1, 7]})
    for model in (str(tmp_path / "bare"), str(tmp_path / "bare" / "config.json")):
        out = tmp_path / ("out_" + os.path.basename(model))
        proc = subprocess.run(
            [os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--random-weights", "--seed", "9", "--weight-std", "0.05",
             "--dtype", "float32", "--out", str(out), "--max-tokens", str(live_token_need(steps))],
            input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        check(collect_logits(steps, str(out), ALL["B"][0]["vocab_size"]), written, reqs, "float32", "random weights")


def test_the_command_reports_bad_models(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(dict(ALL["A"][0], architectures=["NopeForCausalLM"])))
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", "float32", "--out",
         str(tmp_path / "o"), "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0 and "NopeForCausalLM" in proc.stderr
