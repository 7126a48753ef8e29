"""Generation through the entry points: Python engine and command line."""
import json
import os
import subprocess

import pytest
import torch

import plain_llama as P
from tiny_models import ALL, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_model_dir(root, name, seed=21) for name in ("A", "B", "F")}


def engine(model_dir, name, **kw):
    from photon_infer_amd import ContinuousBatchEngine
    opts = dict(dtype="float32", block_size=ALL[name][1]["block_size"], num_blocks=128, max_batch=4)
    opts.update(kw)
    return ContinuousBatchEngine(model_dir, **opts)


def test_greedy_generation_equals_the_plain_implementation(model_dirs):
    # the first tiny benchmark workload: prompts of 5, 9 and 17 tokens, 8 greedy tokens each
    cfg, W = P.read_model_folder(model_dirs["A"])
    prompts = [random_tokens(n, 256, 30 + n) for n in (5, 9, 17)]
    want = [P.greedy_generate(cfg, W, p, 8) for p in prompts]
    eng = engine(model_dirs["A"], "A")
    assert eng.generate(prompts, max_new_tokens=8, ignore_eos=True) == want
    # alone, one at a time: the same tokens as batched with the others
    for p, w in zip(prompts, want):
        assert engine(model_dirs["A"], "A").generate([p], max_new_tokens=8, ignore_eos=True) == [w]
    assert eng.runner.cache.num_live == 0 and eng.runner.cache.free_pages() == 128


@pytest.mark.parametrize("name", ["B", "F"])
def test_greedy_generation_in_bfloat16_follows_the_plain_arg_max(model_dirs, name):
    # F: the kernels chosen at real sizes (products split over k, the two-kernel sampler), through
    # the default engine: graphs and a step ahead
    cfg, W = P.read_model_folder(model_dirs[name])
    prompts = [random_tokens(n, ALL[name][0]["vocab_size"], 40 + n) for n in (1, 7, 33)]
    eng = engine(model_dirs[name], name, dtype="bfloat16", chunk_size=16)
    outs = eng.generate(prompts, max_new_tokens=10, ignore_eos=True)
    assert eng.runner.graph_safe and eng.runner._graphs
    if name == "F":
        counts = eng.runner.workspace.counts
        assert counts["deferred"] > 0 and counts["qkv_pieces"] > 0 and counts["added_by_norm"] > 0, counts
    for p, out in zip(prompts, outs):
        seq = list(p)
        assert len(out) == 10
        for tok in out:
            ref = P.llama_forward(cfg, W, seq)[-1]
            emu = P.llama_forward(cfg, W, seq, act_round=P.bf16_round)[-1]
            slack = 3.0 * (emu - ref).abs().max().item()
            assert ref[tok].item() >= ref.max().item() - 2 * slack, (seq, tok)
            seq.append(tok)


def test_chunked_prefill_beside_decodes_with_temperature(model_dirs):
    # the second tiny benchmark workload: prompts 1, 7, 33, 64, 100 in 16-token chunks
    # beside decodes, 12 tokens each at temperature 0.8
    prompts = [random_tokens(n, 384, 50 + n) for n in (1, 7, 33, 64, 100)]

    def run(order, **kw):
        eng = engine(model_dirs["B"], "B", chunk_size=16, max_step_tokens=40, **kw)
        ids = {i: eng.add_request(prompts[i], 12, temperature=0.8, seed=1000 + i, ignore_eos=True) for i in order}
        eng.run_until_complete()
        return {i: eng.get_result(ids[i]) for i in order}, eng

    a, eng = run([0, 1, 2, 3, 4])
    assert all(len(v) == 12 for v in a.values())
    assert eng.get_stats().num_steps > 12                       # prompts were cut into portions
    b, _ = run([4, 2, 0, 3, 1])                                 # another admission order, other batches
    c, _ = run([3], max_batch=1)                                # alone
    assert a == b and c[3] == a[3]                              # same (seed, request) => same tokens
    # and the draws are those of the plain sampler on the plain logits
    cfg, W = P.read_model_folder(model_dirs["B"])
    from photon_infer_amd.sampling import uniform_draw
    seq = list(prompts[1])
    for k, tok in enumerate(a[1]):
        logits = P.llama_forward(cfg, W, seq)[-1]
        assert tok == P.sample_temperature(logits, 0.8, uniform_draw(1001, k))
        seq.append(tok)


def test_out_of_pages_preempts_and_recomputes_to_the_same_tokens(model_dirs):
    prompts = [random_tokens(n, 256, 60 + n) for n in (20, 20, 20)]
    roomy = engine(model_dirs["A"], "A")
    want = roomy.generate(prompts, max_new_tokens=30, ignore_eos=True)
    tight = engine(model_dirs["A"], "A", num_blocks=30)        # 120 tokens of cache for 3 x 50
    got = tight.generate(prompts, max_new_tokens=30, ignore_eos=True)
    assert tight.get_stats().num_preemptions > 0
    assert got == want
    assert tight.runner.cache.free_pages() == 30
    tight.runner.cache.check_invariants()


def test_eos_ends_a_request_and_limits_hold(model_dirs, tmp_path):
    cfg, W = P.read_model_folder(model_dirs["A"])
    prompt = random_tokens(9, 256, 70)
    free_run = P.greedy_generate(cfg, W, prompt, 8)
    eos = free_run[3]
    d = str(tmp_path / "with_eos")
    os.makedirs(d)
    json.dump(dict(cfg, eos_token_id=[eos, 999999]), open(os.path.join(d, "config.json"), "w"))
    os.symlink(os.path.join(model_dirs["A"], "model.safetensors"), os.path.join(d, "model.safetensors"))
    eng = engine(d, "A")
    rid = eng.add_request(prompt, 8)
    eng.run_until_complete()
    req = eng.get_request(rid)
    assert req.generated_tokens == free_run[:free_run.index(eos) + 1] and req.finish_reason == "eos"
    from photon_infer_amd import RequestError
    with pytest.raises(RequestError, match="vocabulary"):
        eng.add_request([1, 2, 256])
    with pytest.raises(RequestError, match="longer"):
        eng.add_request([1] * 129)


def test_command_line(model_dirs, tmp_path):
    cfg, W = P.read_model_folder(model_dirs["A"])
    prompt = random_tokens(6, 256, 80)
    want = P.greedy_generate(cfg, W, prompt, 5)
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "llama_infer"), model_dirs["A"], "--dtype", "fp32", "--prompt-ids",
         ",".join(map(str, prompt)), "--max-new-tokens", "5", "--temperature", "0", "--block-size", "4", "--ignore-eos"],
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "PhotonInfer - LLaMA Inference Demo" in proc.stdout and "tokens/s" in proc.stdout
    assert f"Generated ids: {','.join(map(str, want))}" in proc.stdout
    # random-weights mode from a bare config.json, text prompt through a tokenizer file
    import base64
    (tmp_path / "cfg").mkdir()
    json.dump(ALL["A"][0], open(tmp_path / "cfg" / "config.json", "w"))
    (tmp_path / "tok.model").write_text("".join(f"{base64.b64encode(bytes([b])).decode()} {b}\n" for b in range(256)))
    cfg_small = dict(ALL["A"][0], vocab_size=128256)
    json.dump(cfg_small, open(tmp_path / "cfg" / "config.json", "w"))
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "llama_infer"), str(tmp_path / "cfg"), str(tmp_path / "tok.model"), "cuda",
         "--random-weights", "--seed", "3", "--prompt", "hi there", "--max-new-tokens", "4"],
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "User: hi there" in proc.stdout and "Prompt tokens: 9" in proc.stdout and "Assistant:" in proc.stdout


@pytest.mark.parametrize("dtype,name", [("float32", "A"), ("bfloat16", "D"), ("bfloat16", "F")])
def test_graph_replayed_decode_equals_eager_steps(tmp_path, dtype, name):
    """Decode-only steps replay a captured graph (model + sampling kernel); every replay must
    give what the eager step gives, with eager work (new requests' prompts) between replays."""
    d = make_model_dir(tmp_path, name, seed=31)
    vocab = ALL[name][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 90 + n) for n in (3, 40, 17, 9)]

    def run(use_graphs):
        eng = engine(d, name, dtype=dtype, use_graphs=use_graphs, chunk_size=8, max_step_tokens=24)
        ids = [eng.add_request(p, 14 + 3 * i, temperature=0.7 if i % 2 else 0.0, seed=7 + i, ignore_eos=True)
               for i, p in enumerate(prompts[:3])]
        for _ in range(12):
            eng.step()
        ids.append(eng.add_request(prompts[3], 9, ignore_eos=True))     # arrives mid-run: eager steps between replays
        eng.run_until_complete()
        return [eng.get_result(i) for i in ids], eng

    eager, _ = run(False)
    graphed, eng = run(True)
    assert eng.runner._graphs, "no decode step went through a graph"
    assert all(g.graph is not None for g in eng.runner._graphs.values())
    assert graphed == eager
    assert [len(x) for x in graphed] == [14, 17, 20, 9]


@pytest.mark.parametrize("name,copies", [("F", 9), ("D", 6), ("E", 2)])
def test_streaming_copies_of_the_weights_change_no_token(tmp_path, name, copies):
    """By default the runner keeps a second copy of every matrix that decode steps stream, in the
    order the kernels load it; a model generates the same tokens with and without (F: all four
    matrices of both layers and the tied head; D: the down projection's 272 columns and the head's
    520 rows do not fit the layout's blocks of 16 x 64, the other three per layer do; E, hidden
    size 160: only the o projection, 160 x 512)."""
    d = make_model_dir(tmp_path, name, seed=33)
    vocab = ALL[name][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 50 + n) for n in (3, 40, 140)]

    def run(stream_copies):
        eng = engine(d, name, dtype="bfloat16", stream_copies=stream_copies, chunk_size=64, max_step_tokens=96)
        out = eng.generate(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True)
        return out, eng

    plain, eng0 = run(False)
    copied, eng1 = run(True)
    assert eng0.runner.stream_copies == 0 and eng1.runner.stream_copies == copies
    assert copied == plain


@pytest.mark.parametrize("dtype,name", [("float32", "A"), ("bfloat16", "D"), ("bfloat16", "F")])
def test_a_step_ahead_gives_the_same_tokens(tmp_path, dtype, name):
    """Launching the next decode step before this one's tokens are on the host (they are fed
    back on the device) changes nothing: requests of different lengths ending at different
    steps, greedy and sampled, one arriving mid-run."""
    d = make_model_dir(tmp_path, name, seed=33)
    vocab = ALL[name][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 70 + n) for n in (4, 21, 9, 15)]

    def run(lookahead):
        eng = engine(d, name, dtype=dtype, lookahead=lookahead, chunk_size=8, max_step_tokens=32)
        ids = [eng.add_request(p, 5 + 6 * i, temperature=0.9 if i % 2 else 0.0, seed=3 + i, ignore_eos=True)
               for i, p in enumerate(prompts[:3])]
        for _ in range(9):
            eng.step()
        ids.append(eng.add_request(prompts[3], 11, temperature=0.5, seed=9, ignore_eos=True))
        eng.run_until_complete()
        assert eng.runner.cache.num_live == 0 and eng.get_stats().num_finished == 4
        eng.runner.cache.check_invariants()
        return [eng.get_result(i) for i in ids]

    plain, ahead = run(False), run(True)
    assert ahead == plain
    assert [len(x) for x in ahead] == [5, 11, 17, 11]


def test_an_end_token_during_a_step_ahead(tmp_path):
    """An end token is only seen one step late: the request's row in the step already launched
    is wasted, its result must not be, and its pages go back when that step has been read."""
    d = make_model_dir(tmp_path, "A", seed=35)
    prompts = [random_tokens(n, 256, 80 + n) for n in (6, 13, 3)]
    free = engine(d, "A", lookahead=False).generate(prompts, max_new_tokens=12, ignore_eos=True)
    # an end token that the second request produces mid-way and that cuts it short
    stop = free[1][5]
    cut = free[1].index(stop) + 1

    def run(lookahead):
        eng = engine(d, "A", lookahead=lookahead)
        eng.eos_token_ids = (stop,)
        ids = [eng.add_request(p, 12) for p in prompts]
        eng.run_until_complete()
        assert eng.runner.cache.num_live == 0 and eng.runner.cache.free_pages() == 128
        eng.runner.cache.check_invariants()
        return [eng.get_result(i) for i in ids], [eng.get_request(i).finish_reason for i in ids]

    (plain, why_plain), (ahead, why_ahead) = run(False), run(True)
    assert ahead == plain and why_ahead == why_plain
    assert ahead[1] == free[1][:cut] and why_ahead[1] == "eos"
    for i in (0, 2):                       # the others run on unless they meet the token themselves
        n = free[i].index(stop) + 1 if stop in free[i] else 12
        assert ahead[i] == free[i][:n]


def test_decode_steps_queued_far_ahead_of_the_gpu(tmp_path):
    """A caller may queue several decode steps without reading any result while the GPU is
    still busy with earlier work: every step must still see its own positions and tables
    (the metadata staging is reused only after its copy has run)."""
    from photon_infer_amd.engine import StepEntry

    d = make_model_dir(tmp_path, "D", seed=37)
    vocab = ALL["D"][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, 60 + n) for n in (5, 18, 11)]
    fed = [random_tokens(7, vocab, 50 + i) for i in range(3)]          # the tokens fed at each decode step, fixed

    def run(busy):
        runner = engine(d, "D", dtype="bfloat16").runner
        rids = [f"r{i}" for i in range(3)]
        for rid, p in zip(rids, prompts):
            runner.admit(rid)
            runner.step([StepEntry(rid, p, [])])
        outs = []
        for s in range(7):
            if s == 1:                                                 # step 0 captured the graph (and drained the GPU)
                torch.cuda.synchronize()
                if busy:
                    torch.cuda._sleep(400_000_000)                     # the GPU stays behind the host for a while
            ids = runner.decode_step([StepEntry(rid, [fed[i][s]], [0]) for i, rid in enumerate(rids)], [0.0] * 3, [0.0] * 3)
            outs.append(ids.clone())
            if not busy:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        return [o.tolist() for o in outs]

    assert run(True) == run(False)


@pytest.mark.parametrize("lookahead", [False, True])
def test_abort_of_waiting_running_and_launched_requests(model_dirs, lookahead):
    """A cancelled request gives its slot and pages back at once, wherever it is: still waiting,
    in the middle of its prompt, decoding, or in a decode step that was launched and not read.
    The others generate what they generate without it; no page or slot is lost."""
    prompts = [random_tokens(n, 256, 160 + n) for n in (6, 30, 11, 4, 9)]
    want = engine(model_dirs["A"], "A", max_batch=3).generate(prompts, max_new_tokens=16, ignore_eos=True)
    eng = engine(model_dirs["A"], "A", max_batch=3, chunk_size=8, max_step_tokens=12, lookahead=lookahead)
    ids = [eng.add_request(p, 16, ignore_eos=True) for p in prompts]
    eng.step()                                               # 0 through, 1 mid-prompt, 3 and 4 waiting (three slots)
    r1 = eng.get_request(ids[1])
    assert 0 < r1.num_computed_tokens < 30 and eng.get_request(ids[4]).state.value == "waiting"
    free = eng.runner.cache.free_pages()
    assert eng.abort(ids[1]) and eng.abort(ids[4])           # mid-prompt, and waiting
    assert eng.runner.cache.free_pages() > free and r1.finish_reason == "aborted" and r1.generated_tokens == []
    eng.runner.cache.check_invariants()
    for _ in range(8):
        eng.step()
    r0 = eng.get_request(ids[0])
    assert not r0.is_finished() and r0.num_generated() > 2
    if lookahead:
        assert eng._in_flight is not None and r0 in eng._in_flight.reqs      # a step with it is on the GPU, unread
    had, live = list(r0.generated_tokens), eng.runner.cache.num_live
    assert eng.abort(ids[0])
    assert eng.runner.cache.num_live == live - 1             # before the launched step is read
    eng.runner.cache.check_invariants()
    eng.run_until_complete()
    assert r0.generated_tokens == had == want[0][:len(had)] and r0.finish_reason == "aborted"
    assert eng.get_result(ids[2]) == want[2] and eng.get_result(ids[3]) == want[3]
    assert not eng.abort(ids[2])                             # finished long ago
    assert eng.runner.cache.num_live == 0 and eng.runner.cache.free_pages() == 128
    eng.runner.cache.check_invariants()
    assert eng.get_stats().num_aborted == 3


def test_the_default_pool_fits_the_device_and_too_much_is_a_typed_error(tmp_path):
    """Without a pool size the engine takes every slot at the model's full length if that fits,
    else a share of the memory that is free after the weights, and lets no sequence grow beyond
    it; a size that was asked for and does not fit is an error of the engine's own, before any
    allocation."""
    from photon_infer_amd import ContinuousBatchEngine, ErrorCode, OutOfMemoryError, write_random_model
    from photon_infer_amd.config import LlamaConfig
    huge = LlamaConfig.from_dict(dict(ALL["A"][0], max_position_embeddings=1 << 30))
    d = write_random_model(huge, str(tmp_path / "huge"), seed=1, std=0.02)
    free, _ = torch.cuda.mem_get_info()
    eng = ContinuousBatchEngine(d, dtype="bfloat16", block_size=16, max_batch=8, memory_fraction=0.02)
    page_bytes = 2 * 2 * (2 * 16 * 16) * 2                  # layers x (k, v) x kv heads x head size x page x bytes
    pool = eng.runner.num_pages * page_bytes
    assert 0.01 * free < pool <= 0.021 * free
    assert eng.runner.max_model_len == eng.runner.num_pages * 16 < (1 << 30)
    assert eng.generate([[1, 2, 3]], max_new_tokens=4, ignore_eos=True)[0].__len__() == 4
    del eng
    small = ContinuousBatchEngine(d, dtype="bfloat16", block_size=16, max_batch=2, max_model_len=256)
    assert small.runner.num_pages == 2 * 256 // 16 and small.runner.max_model_len == 256     # fits: every slot at full length
    with pytest.raises(OutOfMemoryError, match="num_blocks=") as err:
        ContinuousBatchEngine(d, dtype="bfloat16", block_size=16, num_blocks=1 << 34)
    assert err.value.code == ErrorCode.OUT_OF_MEMORY and "GiB" in str(err.value)
    with pytest.raises(OutOfMemoryError, match="max_cache_tokens="):
        ContinuousBatchEngine(d, dtype="bfloat16", block_size=16, max_cache_tokens=1 << 40)


def test_two_engines_stepping_in_turns_do_not_disturb_each_other(model_dirs):
    """Every runner owns its kernel scratch and its pending residual update: two engines in one
    process, stepped alternately (as two threads would interleave), generate what each generates
    alone.  Model F leaves a product in pieces at the end of nearly every kernel sequence."""
    prompts_a = [random_tokens(n, 32768, 140 + n) for n in (5, 40, 17)]
    prompts_b = [random_tokens(n, 32768, 150 + n) for n in (23, 3)]

    def make():
        return engine(model_dirs["F"], "F", dtype="bfloat16", chunk_size=16, max_step_tokens=24)

    alone_a = make().generate(prompts_a, max_new_tokens=12, temperature=0.7, seed=5, ignore_eos=True)
    alone_b = make().generate(prompts_b, max_new_tokens=15, temperature=0.7, seed=9, ignore_eos=True)
    ea, eb = make(), make()
    assert ea.runner.workspace is not eb.runner.workspace
    ids_a = [ea.add_request(p, 12, temperature=0.7, seed=5 + i, ignore_eos=True) for i, p in enumerate(prompts_a)]
    ids_b = [eb.add_request(p, 15, temperature=0.7, seed=9 + i, ignore_eos=True) for i, p in enumerate(prompts_b)]
    while ea.has_work() or eb.has_work():
        if ea.has_work():
            ea.step()
        if eb.has_work():
            eb.step()
    assert [ea.get_result(i) for i in ids_a] == alone_a
    assert [eb.get_result(i) for i in ids_b] == alone_b


def test_cpp_program_generates_what_the_python_entry_point_generates(model_dirs, tmp_path):
    """The library API for C and C++ programs drives the same engine: a C++ program built
    against it generates the same tokens for the same requests."""
    import cpp_api

    prompts = [random_tokens(n, 256, 40 + n) for n in (5, 12, 3)]
    want = engine(model_dirs["A"], "A").generate(prompts, max_new_tokens=9, ignore_eos=True)
    exe = cpp_api.build_demo(tmp_path)
    r = cpp_api.run_demo(exe, model_dirs["A"], "float32", ";".join(",".join(map(str, p)) for p in prompts), 9,
                         ALL["A"][1]["block_size"])
    assert r.returncode == 0, (r.stdout, r.stderr)
    got = [[int(t) for t in line.split()] for line in r.stdout.strip().splitlines()]
    assert got == want


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16")])
def test_random_workloads_do_not_depend_on_graphs_or_on_running_ahead(tmp_path, name, dtype):
    """Seeded random workloads (prompt and output lengths, temperatures, arrival steps, pool
    and batch sizes small enough to force preemption): the tokens and the reasons for ending
    are the same with and without graphs, with and without the step ahead, and no page or
    slot is lost."""
    import random

    d = make_model_dir(tmp_path, name, seed=41)
    vocab, block = ALL[name][0]["vocab_size"], ALL[name][1]["block_size"]
    for seed in range(4):
        rng = random.Random(1000 * seed + len(name))
        n = rng.randint(3, 8)
        reqs = [(random_tokens(rng.randint(1, 50), vocab, 100 * seed + i), rng.randint(1, 20), rng.choice([0.0, 0.0, 0.7, 1.1]),
                 rng.randint(0, 25)) for i in range(n)]
        opts = dict(num_blocks=rng.choice([12, 20, 40, 128]), max_batch=rng.choice([2, 3, 4, 6]), chunk_size=rng.choice([4, 8, 16]),
                    max_step_tokens=rng.choice([8, 16, 32]))    # one product kernel serves steps up to 32 tokens: the same bits
        outcomes = {}
        for lookahead, graphs in ((False, False), (False, True), (True, True)):
            eng = engine(d, name, dtype=dtype, block_size=block, lookahead=lookahead, use_graphs=graphs, **opts)
            waiting, ids, step = sorted(range(n), key=lambda i: reqs[i][3]), {}, 0
            while waiting or eng.has_work():
                while waiting and reqs[waiting[0]][3] <= step:
                    i = waiting.pop(0)
                    ids[i] = eng.add_request(reqs[i][0], reqs[i][1], temperature=reqs[i][2], seed=seed + i, ignore_eos=seed % 2 == 0)
                eng.step()
                step += 1
                assert step < 3000, "the engine makes no progress"
            eng.runner.cache.check_invariants()
            assert eng.runner.cache.num_live == 0
            outcomes[(lookahead, graphs)] = [(eng.get_result(ids[i]), eng.get_request(ids[i]).finish_reason) for i in range(n)]
        assert outcomes[(False, True)] == outcomes[(False, False)], (seed, opts)
        assert outcomes[(True, True)] == outcomes[(False, False)], (seed, opts)
