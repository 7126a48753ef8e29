"""The paths that the benchmark times, under a comparison.

Decode steps replayed from graphs whose attention is cut into several key ranges (contexts past
128, 256 and 512 tokens, the ranges merged by the o projection), the switch from one length
bucket's graph to the next, the step launched ahead - against eager steps and against the plain
implementation; and the chain of kernels that runs at the benchmark's own layer sizes (hidden
2,048, intermediate 8,192, 32 heads on 8 of 64, a vocabulary of 128,256), two layers of it,
against the plain implementation: a 2,048-token prompt whole, then decode steps of batch 8.
"""
import pytest
import torch

import plain_llama as P
import plain_wide as PW
from tiny_models import ALL, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

# batch size -> (prompt lengths, new tokens): contexts cross 128, 256 and 512 while decoding
CASES = {
    1: ([120], [140]),
    3: ([100, 250, 490], [40, 60, 80]),
    8: ([100, 118, 230, 250, 300, 470, 490, 60], [60, 40, 50, 80, 40, 60, 45, 70]),
}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_model_dir(root, name, seed=51) for name in ("D", "F")}


def engine(model_dir, name, **kw):
    from photon_infer_amd import ContinuousBatchEngine
    opts = dict(dtype="bfloat16", block_size=16, num_blocks=256, max_batch=8, max_model_len=1024, chunk_size=128,
                max_step_tokens=256)
    opts.update(kw)
    return ContinuousBatchEngine(model_dir, **opts)


def generate(eng, prompts, new_tokens, temperatures):
    ids = [eng.add_request(p, n, temperature=t, seed=11 + i, ignore_eos=True)
           for i, (p, n, t) in enumerate(zip(prompts, new_tokens, temperatures))]
    eng.run_until_complete()
    assert eng.runner.cache.num_live == 0
    eng.runner.cache.check_invariants()
    return [eng.get_result(i) for i in ids]


@pytest.mark.parametrize("batch", [1, 3, 8])
@pytest.mark.parametrize("name", ["D", "F"])
def test_graphs_over_several_key_ranges_equal_eager_steps(model_dirs, name, batch):
    """Greedy and sampled requests whose contexts pass 128, 256 and 512 tokens while they decode:
    every decode step's attention is cut into key ranges that the o projection merges, one graph
    per (batch size, length bucket) is captured and left behind, and the tokens are those of the
    same steps launched kernel by kernel; launching a step ahead changes nothing either (every
    request is there from the start and ends by its length, so the batches are the same)."""
    lengths, new_tokens = CASES[batch]
    vocab = ALL[name][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 300 + n) for n in lengths]
    temps = [0.0 if i % 2 == 0 else 0.8 for i in range(batch)]

    def run(use_graphs, lookahead):
        eng = engine(model_dirs[name], name, use_graphs=use_graphs, lookahead=lookahead)
        return generate(eng, prompts, new_tokens, temps), eng

    eager, e0 = run(False, False)
    graphed, e1 = run(True, False)
    ahead, e2 = run(True, True)
    assert [len(x) for x in eager] == new_tokens
    assert not e0.runner._graphs and len(e1.runner._graphs) >= 3, sorted(e1.runner._graphs)
    assert len({bucket for _, bucket in e1.runner._graphs}) >= 2          # more than one length bucket was decoded in
    assert all(g.graph is not None for g in e1.runner._graphs.values())
    for e in (e0, e1, e2):
        assert e.runner.workspace.counts["ranges_merged_by_product"] > 0, e.runner.workspace.counts
    assert graphed == eager
    assert ahead == eager


@pytest.mark.parametrize("name", ["D", "F"])
def test_greedy_decoding_past_several_buckets_follows_the_plain_arg_max(model_dirs, name):
    """The same requests, greedy, through the default engine (graphs, a step ahead): every token
    is the plain implementation's arg max, or within the slack that bfloat16 rounding leaves
    between two candidates."""
    lengths, new_tokens = CASES[3]
    vocab = ALL[name][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 300 + n) for n in lengths]
    eng = engine(model_dirs[name], name)
    outs = generate(eng, prompts, new_tokens, [0.0] * 3)
    assert len(eng.runner._graphs) >= 3 and eng.runner.workspace.counts["ranges_merged_by_product"] > 0
    cfg, W = P.read_model_folder(model_dirs[name])
    for p, out in zip(prompts, outs):
        seq = list(p) + list(out)
        rows = list(range(len(p) - 1, len(seq) - 1))                     # the rows that chose the new tokens
        ref = PW.llama_forward(cfg, W, seq, rows, device="cuda").cpu()
        emu = PW.llama_forward(cfg, W, seq, rows, act_round=P.bf16_round, device="cuda").cpu()
        slack = 3.0 * (emu - ref).abs().max().item()
        for k, tok in enumerate(out):
            assert ref[k, tok].item() >= ref[k].max().item() - 2 * slack, (len(p), k, tok)


# ------------------------------------------------------------------ the benchmarks' layer sizes
_LLAMA3 = dict(rope_type="llama3", low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
BENCH_SIZES = {
    # Llama 3.2 1B, 3.2 3B (three heads per kv head, head size 128) and 3.1 8B (untied head) layer sizes, two layers each
    "1b": dict(hidden_size=2048, intermediate_size=8192, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               tie_word_embeddings=True, rope_scaling=dict(_LLAMA3, factor=32.0)),
    "3b": dict(hidden_size=3072, intermediate_size=8192, num_attention_heads=24, num_key_value_heads=8, head_dim=128,
               tie_word_embeddings=True, rope_scaling=dict(_LLAMA3, factor=32.0)),
    "8b": dict(hidden_size=4096, intermediate_size=14336, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               tie_word_embeddings=False, rope_scaling=dict(_LLAMA3, factor=8.0)),
}


@pytest.mark.parametrize("size", ["1b", "3b", "8b"])
def test_two_layers_at_the_benchmark_sizes_against_the_plain_implementation(monkeypatch, size):
    """What ``bench.py`` times, compared: a 2,048-token prompt in one step (at 1B sizes the large-tile
    product fed k in four pieces, the o projection in pieces, prompt attention over 16 rounds), then
    16 decode steps of batch 8 through ``decode_step`` (graphs of the 4,096 bucket: eight key ranges,
    merged by the o projection where its matrix is small enough, every product streamed in pieces,
    the output head over 128,256 rows, the two-kernel sampler), logits of the prompts' last rows and
    of every decode row against the plain implementation.  The 3B and 8B sizes are those of the
    continuous-batching and mixed-step workloads: head size 128, three and four heads per kv head."""
    from photon_infer_amd.config import LlamaConfig
    from photon_infer_amd.engine import EngineOptions, ModelRunner, StepEntry
    from photon_infer_amd.ops import fast
    from photon_infer_amd.registry import build_model_spec

    cfg = LlamaConfig.from_dict(dict(BENCH_SIZES[size], architectures=["LlamaForCausalLM"], num_hidden_layers=2, vocab_size=128256,
                                     max_position_embeddings=131072, rms_norm_eps=1e-5, rope_theta=500000.0))
    spec = build_model_spec(cfg)
    gen = torch.Generator(device="cuda").manual_seed(5)
    tensors = {}
    for s in spec.tensor_specs():
        if s.role == "norm":
            t = torch.rand(s.shape, generator=gen, device="cuda") + 0.5
        else:
            t = torch.randn(s.shape, generator=gen, device="cuda") * 0.02
        tensors[s.name] = t.to(torch.bfloat16)
    plain_weights = dict(tensors)

    calls = {"tile": [], "skinny": []}
    tile_splits, skinny_splits = fast._tile_splits, fast._skinny_splits
    monkeypatch.setattr(fast, "_tile_splits", lambda M, N, K: calls["tile"].append((M, N, K, tile_splits(M, N, K))) or calls["tile"][-1][3])
    monkeypatch.setattr(fast, "_skinny_splits", lambda M, N, K: calls["skinny"].append((M, N, K, skinny_splits(M, N, K))) or calls["skinny"][-1][3])

    lengths = [2048, 1500, 900, 400, 130, 2000, 64, 1024]
    steps = 16
    runner = ModelRunner(None, EngineOptions(max_batch=8, max_cache_tokens=8 * (2048 + 64), max_model_len=4096, keep_logits=True),
                         config=cfg, tensors=tensors)
    assert runner.stream_copies == 9 and runner.graph_safe                # four matrices per layer and the head (or the embedding it is tied to)
    prompts = [random_tokens(n, cfg.vocab_size, 500 + n) for n in lengths]
    rids = [f"r{i}" for i in range(8)]
    got = [[] for _ in rids]                                  # per request: logits rows, the prompt's last first
    seqs = [list(p) for p in prompts]
    for i, (rid, p) in enumerate(zip(rids, prompts)):
        runner.admit(rid)
        logits = runner.step([StepEntry(rid, p, [len(p) - 1])])
        got[i].append(logits[0].cpu())
        seqs[i].append(int(logits[0].argmax()))
    if size == "1b":
        assert (2048, 2048, 8192, 4) in calls["tile"], calls["tile"]          # the down projection of the whole prompt
    for _ in range(steps):
        ids = runner.decode_step([StepEntry(rid, [seq[-1]], [0]) for rid, seq in zip(rids, seqs)], [0.0] * 8, [0.0] * 8)
        logits = runner.decode_logits.cpu()
        for i, tok in enumerate(ids.tolist()):
            got[i].append(logits[i].clone())
            assert tok == int(logits[i].argmax())             # the graph's sampler chose this row's first maximum
            seqs[i].append(tok)
    assert list(runner._graphs) == [(8, 4096)]
    counts = runner.workspace.counts
    # (counted where Python launches: the eager first step and the capture, not the replays)
    assert counts["qkv_pieces"] > 0 and counts["added_by_norm"] > 0 and counts["deferred"] > 0, counts
    D, I = cfg.hidden_size, cfg.intermediate_size
    assert any(c[:3] == (8, D, cfg.q_size) and c[3] > 1 for c in calls["skinny"]), set(calls["skinny"])     # o, in pieces
    assert any(c[:3] == (8, D, I) and c[3] > 1 for c in calls["skinny"]), set(calls["skinny"])              # down, in pieces
    if size == "1b":
        assert counts["ranges_merged_by_product"] >= 2
        assert (8, 2048, 2048, 8) in calls["skinny"] and (8, 2048, 8192, 8) in calls["skinny"], set(calls["skinny"])
    elif size == "8b":
        assert counts["ranges_merged_by_product"] == 0        # its o matrix (32 MB) is streamed by the plain kernel, the ranges merged before
    # one mixed step on top: a 300-token portion for the request that is 146 tokens long, a
    # 40-token one for the longest, single tokens for the rest (the tile kernel and the key-split
    # kernel share the step; the portions' products take the tile kernels, fed late in a context)
    more = {4: random_tokens(300, cfg.vocab_size, 901), 0: random_tokens(40, cfg.vocab_size, 902)}
    entries, fed = [], []
    for i, rid in enumerate(rids):
        toks = [seqs[i][-1]] + more[i] if i in more else [seqs[i][-1]]
        entries.append(StepEntry(rid, toks, [len(toks) - 1]))
        fed.append(toks)
    mixed = runner.step(entries).cpu()
    for rid in rids:
        runner.release(rid)
    assert runner.cache.free_pages() == runner.num_pages

    raw = cfg.to_dict()
    for i, p in enumerate(prompts):
        seq = seqs[i][:-1] + fed[i]                           # everything that was fed
        rows = list(range(len(p) - 1, len(seqs[i]) - 1)) + [len(seq) - 1]
        assert len(rows) == steps + 2 == len(got[i]) + 1
        ref = PW.llama_forward(raw, plain_weights, seq, rows, device="cuda").cpu()
        emu = PW.llama_forward(raw, plain_weights, seq, rows, act_round=P.bf16_round, device="cuda").cpu()
        tol = 3.0 * (emu - ref).abs().max().item()
        err = max((g - r).abs().max().item() for g, r in zip(got[i] + [mixed[i]], ref))
        assert err <= tol, (i, len(p), err, tol)
        assert tol < 0.2 * ref.abs().max().item()             # the yardstick itself is tight


def test_float32_decoding_over_key_ranges_equals_the_plain_implementation(model_dirs):
    """The float32 path at contexts where its attention kernel cuts a decoding token's keys into
    ranges (from 256 keys on) and its products take the weight-streaming kernel for few rows:
    single tokens through ``step`` and through ``decode_step`` (a replayed graph) give the same
    logits bit for bit, and they are the plain implementation's."""
    from photon_infer_amd import ops
    from photon_infer_amd.engine import EngineOptions, ModelRunner, StepEntry
    cfg, W = P.read_model_folder(model_dirs["D"])
    vocab = ALL["D"][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 700 + n) for n in (300, 530, 40)]
    steps = 24
    assert ops.general_attention_ranges(3, ALL["D"][0]["num_attention_heads"], 531) > 1

    def run(graphs):
        runner = ModelRunner(model_dirs["D"], EngineOptions(dtype="float32", block_size=16, num_blocks=96, max_batch=3,
                                                            use_graphs=graphs, keep_logits=True))
        seqs, rows = [list(p) for p in prompts], [[] for _ in prompts]
        for i, p in enumerate(prompts):
            runner.admit(i)
            logits = runner.step([StepEntry(i, p, [len(p) - 1])])
            rows[i].append(logits[0].cpu())
            seqs[i].append(int(logits[0].argmax()))
        for _ in range(steps):
            entries = [StepEntry(i, [s[-1]], [0]) for i, s in enumerate(seqs)]
            if graphs:
                ids = runner.decode_step(entries, [0.0] * 3, [0.0] * 3).tolist()
                logits = runner.decode_logits.cpu()
            else:
                logits = runner.step(entries).cpu()
                ids = [int(r.argmax()) for r in logits]
            for i, tok in enumerate(ids):
                rows[i].append(logits[i].clone())
                seqs[i].append(tok)
        assert bool(runner._graphs) == graphs
        return seqs, rows

    seqs, eager = run(False)
    seqs_g, graphed = run(True)
    assert seqs_g == seqs
    for a, b in zip(eager, graphed):
        assert all(torch.equal(x, y) for x, y in zip(a, b))           # the same bits, eagerly and replayed
    for i, p in enumerate(prompts):
        seq = seqs[i][:-1]
        ref = PW.llama_forward(cfg, W, seq, list(range(len(p) - 1, len(seq))), device="cuda").cpu()
        tol = 3e-5 * max(1.0, ref.abs().max().item())
        err = max((g - r).abs().max().item() for g, r in zip(eager[i], ref))
        assert err <= tol, (i, err, tol)
