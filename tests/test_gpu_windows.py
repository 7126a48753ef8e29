"""A model whose layers keep different amounts of the past: one attends to all keys, two to a
window of the last W (two different W, so three cache groups with pools and block tables of
their own).  Defined and registered here, from the framework's own parts; stepped through
``ModelRunner.step`` in every way of cutting, in float32 and in bfloat16, against a plain
implementation from the same functions as the Llama one (tests/plain_llama.py).  While a long
request runs, the windowed groups give pages back as the window passes them and take them again.
"""
import dataclasses
import math

import pytest
import torch

import plain_llama as P
from gpu_tools import bf16_tol, cut_steps, fp32_tol, live_token_need, run_trace
from tiny_models import random_tokens

pytestmark = pytest.mark.gpu

WINDOWS = (None, 40, 24)        # per layer
PAGE = 16


def register_window_toy():
    from photon_infer_amd import register_architecture
    from photon_infer_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, ModelSpec,
                                        TokenEmbedding)

    @dataclasses.dataclass(frozen=True)
    class WindowToyConfig:
        architecture: str
        hidden_size: int
        vocab_size: int
        num_heads: int
        num_kv_heads: int
        head_dim: int
        intermediate_size: int
        eps: float
        windows: tuple
        torch_dtype: str = "bfloat16"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(raw["architectures"][0], raw["hidden_size"], raw["vocab_size"], raw["num_heads"], raw["num_kv_heads"],
                       raw["head_dim"], raw["intermediate_size"], raw["eps"], tuple(raw["windows"]), raw.get("torch_dtype", "bfloat16"))

        def to_dict(self):
            d = dataclasses.asdict(self)
            d["architectures"] = [d.pop("architecture")]
            d["windows"] = list(d["windows"])
            return d

    def build(cfg):
        D = cfg.hidden_size
        rope = POSITION_ENCODINGS.make("rope", head_dim=cfg.head_dim, theta=10000.0)
        layers = []
        for i, w in enumerate(cfg.windows):
            mixer = MIXERS.make("attention", hidden_size=D, num_heads=cfg.num_heads, num_kv_heads=cfg.num_kv_heads,
                                head_dim=cfg.head_dim, position=rope, window=w)
            layers.append((f"layers.{i}.", BLOCKS.make(
                "prenorm", norm1=("n1.", NORMS.make("rmsnorm", dim=D, eps=cfg.eps)), mixer=("attn.", mixer),
                norm2=("n2.", NORMS.make("rmsnorm", dim=D, eps=cfg.eps)),
                ffn=("ffn.", FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=cfg.intermediate_size)))))
        return ModelSpec(hidden_size=D, vocab_size=cfg.vocab_size, max_positions=1024,
                         embedding=("emb.", TokenEmbedding(cfg.vocab_size, D)), layers=layers,
                         final_norm=("norm.", NORMS.make("rmsnorm", dim=D, eps=cfg.eps)),
                         head=("head.", LMHead(cfg.vocab_size, D, tied=True)))

    register_architecture("WindowToyForCausalLM", WindowToyConfig, build)
    return WindowToyConfig


def plain_window_toy(cfg, W, toks, windows=None, act_round=None):
    """The toy on a whole sequence: the Llama layer (tests/plain_llama.py's functions) with a
    window per layer."""
    rd = act_round or (lambda t: t)
    W = {n: t.float() for n, t in W.items()}
    D, nh, nkv, hd, eps = cfg["hidden_size"], cfg["num_heads"], cfg["num_kv_heads"], cfg["head_dim"], cfg["eps"]
    S = len(toks)
    f = P.rope_frequencies(hd, 10000.0, None)
    x = P.embedding(W["emb.weight"], toks)
    for i, w in enumerate(cfg["windows"] if windows is None else windows):
        p = f"layers.{i}."
        h = rd(P.rmsnorm(x, W[p + "n1.weight"], eps))
        q = rd(P.rope(rd(P.linear(h, W[p + "attn.q_proj.weight"])).reshape(S, nh, hd), range(S), f, False))
        k = rd(P.rope(rd(P.linear(h, W[p + "attn.k_proj.weight"])).reshape(S, nkv, hd), range(S), f, False))
        v = rd(P.linear(h, W[p + "attn.v_proj.weight"])).reshape(S, nkv, hd)
        a = rd(P.attention(q, k, v, 1 / math.sqrt(hd), window=w, p_round=act_round).reshape(S, nh * hd))
        x = x + P.linear(a, W[p + "attn.o_proj.weight"])
        h = rd(P.rmsnorm(x, W[p + "n2.weight"], eps))
        x = x + P.linear(rd(P.swiglu(rd(P.linear(h, W[p + "ffn.gate_proj.weight"])), rd(P.linear(h, W[p + "ffn.up_proj.weight"])))),
                         W[p + "ffn.down_proj.weight"])
    return P.linear(rd(P.rmsnorm(x, W["norm.weight"], eps)), W["emb.weight"])


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from photon_infer_amd import write_random_model
    Config = register_window_toy()
    cfg = Config("WindowToyForCausalLM", hidden_size=128, vocab_size=300, num_heads=4, num_kv_heads=2, head_dim=64,
                 intermediate_size=272, eps=1e-5, windows=WINDOWS)
    d = write_random_model(cfg, str(tmp_path_factory.mktemp("window_toy") / "m"), seed=7, std=0.09, norm_init="uniform",
                           dtype="bfloat16")
    raw, W = P.read_model_folder(d)
    return d, raw, W


_plain = {}


def references(toy, toks):
    d, raw, W = toy
    key = tuple(toks)
    if key not in _plain:
        _plain[key] = (plain_window_toy(raw, W, toks), plain_window_toy(raw, W, toks, act_round=P.bf16_round))
    return _plain[key]


def check(got, toy, reqs, dtype, what):
    for rid, toks in reqs.items():
        ref, emu = references(toy, toks)
        tol = fp32_tol(ref) if dtype == "float32" else bf16_tol(ref, emu)
        for p in range(len(toks)):
            err = (got[(rid, p)] - ref[p]).abs().max().item()
            assert err <= tol, f"{what}: {rid} position {p}: error {err:.3e} > {tol:.3e} (first wrong position)"


def runner_for(d, dtype, max_tokens):
    from photon_infer_amd.engine.replay import make_runner
    return make_runner(d, dtype, max_tokens, PAGE)


def test_the_windows_matter_and_the_groups_are_three(toy):
    d, raw, W = toy
    toks = random_tokens(150, 300, 1)
    ref, emu = references(toy, toks)
    no_window = plain_window_toy(raw, W, toks, windows=(None, None, None))
    wrong_edge = plain_window_toy(raw, W, toks, windows=(None, 41, 24))
    tol = bf16_tol(ref, emu)
    assert (no_window[100:] - ref[100:]).abs().max() > 5 * tol      # a kernel that ignored the windows would be caught
    assert (wrong_edge[100:] - ref[100:]).abs().max() > fp32_tol(ref) * 3   # and one key too many, in float32
    runner = runner_for(d, "float32", 64)
    assert [g.window for g in runner.plan.groups] == [None, 24, 40]
    assert [g.owners for g in runner.plan.groups] == [((0, 0),), ((2, 0),), ((1, 0),)]
    assert len({id(lc.k) for lc in runner.layer_caches}) == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_of_a_windowed_model(toy, tmp_path, dtype):
    d = toy[0]
    reqs = {"r0": random_tokens(230, 300, 2)}
    n = 230
    for sizes in ([n], [n - 32] + [1] * 32, [7, 2, 16, 3, 2, 33, 1, 5], [2], [64, 2, 2, 19], [130, 2, 98]):
        steps = cut_steps("r0", reqs["r0"], sizes)
        runner = runner_for(d, dtype, live_token_need(steps))
        check(run_trace(runner, steps, str(tmp_path / f"c{sizes[0]}_{len(sizes)}")), toy, reqs, dtype, f"portions {sizes[:4]}")
        assert runner.cache.num_live == 0
        assert all(runner.cache.free_pages(g) == runner.num_pages for g in range(3))
        runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windowed_groups_give_pages_back_while_the_request_runs(toy, tmp_path, dtype):
    """One long request fed in portions and single tokens: the full group holds a page for every
    16 tokens, the windowed groups only what their window still sees, and the pages they gave back
    are the ones they take next."""
    from photon_infer_amd.engine import StepEntry
    d = toy[0]
    toks = random_tokens(400, 300, 3)
    ref, emu = references(toy, toks)
    tol = fp32_tol(ref) if dtype == "float32" else bf16_tol(ref, emu)
    runner = runner_for(d, dtype, 448)          # 28 pages per group
    runner.admit("a")
    slot = runner.cache.slot("a")
    pos, seen = 0, {1: set(), 2: set()}
    sizes = [50, 1, 1, 30, 2, 1, 1, 1, 64, 1, 1, 17] + [1] * 40 + [100, 3] + [1] * 20 + [64, 3]
    reused, gone = {1: False, 2: False}, {1: set(), 2: set()}
    for n in sizes:
        n = min(n, len(toks) - pos)
        if n == 0:
            break
        logits = runner.step([StepEntry("a", toks[pos:pos + n], list(range(n)))]).cpu()
        for i in range(n):
            err = (logits[i] - ref[pos + i]).abs().max().item()
            assert err <= tol, f"position {pos + i}: error {err:.3e} > {tol:.3e}"
        pos += n
        assert runner.num_pages - runner.cache.free_pages(0) == -(-pos // PAGE)          # the full group keeps all
        for g, window in ((1, 24), (2, 40)):
            held = runner.num_pages - runner.cache.free_pages(g)
            first_needed = max(0, pos - window + 1) // PAGE
            assert held == -(-pos // PAGE) - first_needed <= -(-(window + PAGE) // PAGE) + 1
            row = runner.cache.table_rows(g, [slot])[0]
            now = {int(p) for p in row if p >= 0}
            reused[g] = reused[g] or bool(now & gone[g])       # a page it had given back is in its table again
            seen[g] |= now
            gone[g] = seen[g] - now
        runner.cache.check_invariants()
    assert pos == 400
    # 400 tokens went through groups that never held more than a few pages: pages were used again
    assert len(seen[1]) < 400 // PAGE and len(seen[2]) < 400 // PAGE and reused[1] and reused[2]
    runner.release("a")
    assert all(runner.cache.free_pages(g) == runner.num_pages for g in range(3))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_requests_on_a_windowed_model(toy, tmp_path, dtype):
    from test_gpu_replay import mixed_trace
    d = toy[0]
    lengths = [200, 33, 2, 129, 300, 64, 90]
    reqs = {f"r{i}": random_tokens(n, 300, 40 + i) for i, n in enumerate(lengths)}
    pats = [[16, 1, 1, 1, 2], [1], [33, 2, 7], [64, 1, 1], [5, 3, 2], [2, 2, 50], [1, 1, 1, 40]]
    steps = mixed_trace(reqs, {rid: pats[i % len(pats)] for i, rid in enumerate(reqs)})
    runner = runner_for(d, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), toy, reqs, dtype, "mixed")
    runner.cache.check_invariants()
    assert runner.cache.num_live == 0 and all(runner.cache.free_pages(g) == runner.num_pages for g in range(3))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_engine_with_graphs_on_a_windowed_model(toy, dtype):
    """``ContinuousBatchEngine`` with its default options (decode steps replayed from graphs, a step
    launched ahead) over the three cache groups: the graphs' block tables are as wide as the length
    bucket while the windowed groups' early columns hold no page any more, contexts pass the windows
    and several buckets, requests end at different steps.  The tokens are those of eager steps, the
    greedy ones the plain implementation's arg max, and every page comes back."""
    from photon_infer_amd import ContinuousBatchEngine
    d, raw, W = toy
    prompts = [random_tokens(n, 300, 70 + n) for n in (90, 20, 150, 45)]
    new = [70, 140, 40, 100]                    # contexts reach 160, 160, 190, 145: past both windows and past 128
    temps = [0.0, 0.9, 0.0, 0.7]

    def run(**kw):
        eng = ContinuousBatchEngine(d, dtype=dtype, block_size=PAGE, num_blocks=64, max_batch=4, chunk_size=64,
                                    max_step_tokens=96, **kw)
        ids = [eng.add_request(p, n, temperature=t, seed=5 + i, ignore_eos=True) for i, (p, n, t) in enumerate(zip(prompts, new, temps))]
        eng.run_until_complete()
        assert eng.runner.cache.num_live == 0 and all(eng.runner.cache.free_pages(g) == 64 for g in range(3))
        eng.runner.cache.check_invariants()
        return [eng.get_result(i) for i in ids], eng

    eager, _ = run(use_graphs=False, lookahead=False)
    graphed, eng = run()
    assert eng.runner.graph_safe and len(eng.runner._graphs) >= 3 and len({b for _, b in eng.runner._graphs}) >= 2
    assert graphed == eager
    for p, out, t in zip(prompts, graphed, temps):
        if t > 0:
            continue
        seq = list(p) + list(out)
        ref = plain_window_toy(raw, W, seq)
        emu = plain_window_toy(raw, W, seq, act_round=P.bf16_round) if dtype == "bfloat16" else ref
        slack = 1e-4 if dtype == "float32" else 3.0 * (emu - ref).abs().max().item()
        for k, tok in enumerate(out):
            row = ref[len(p) - 1 + k]
            assert row[tok].item() >= row.max().item() - 2 * slack, (len(p), k, tok)
