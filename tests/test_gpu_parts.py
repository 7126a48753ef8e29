"""Each part alone against the plain implementation, and a toy architecture whose mixer keeps
a state of its own, defined here and registered without touching the framework's files."""
import dataclasses
import json
import math
import os

import pytest
import torch

import plain_llama as P
from gpu_tools import DEV, PagedKV, attention_ctx
from tiny_models import random_tokens

pytestmark = pytest.mark.gpu
F32, BF16 = torch.float32, torch.bfloat16


def gen(seed):
    return torch.Generator().manual_seed(seed)


def load(part, tensors, dtype):
    part.load({k: v.to(dtype).to(DEV) for k, v in tensors.items()}, dtype, torch.device(DEV))
    return part


# ------------------------------------------------------------------ single parts
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_rmsnorm_part(dtype):
    from photon_infer_amd.parts import NORMS
    w = torch.rand(200, generator=gen(0)) + 0.5
    norm = load(NORMS.make("rmsnorm", dim=200, eps=3e-4), {"weight": w}, dtype)
    assert [(s.name, s.shape, s.role) for s in norm.tensor_specs()] == [("weight", (200,), "norm")]
    x = torch.randn(6, 200, generator=gen(1)) * 5
    got = norm.forward(x.to(DEV))
    assert got.dtype == dtype
    want = P.rmsnorm(x, w.to(dtype).float(), 3e-4)
    assert (got.float().cpu() - want).abs().max() <= (1e-5 if dtype == F32 else 2 ** -8 * want.abs().max())


def test_rotary_part_builds_the_plain_frequencies():
    from photon_infer_amd.config import RopeScaling
    from photon_infer_amd.parts import POSITION_ENCODINGS
    sc = dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=8192)
    rope = POSITION_ENCODINGS.make("rope", head_dim=64, theta=500000.0, scaling=RopeScaling(**sc))
    rope.load({}, F32, torch.device(DEV))
    inv, rdim, inter = rope.rotary_params()
    want = torch.tensor(P.rope_frequencies(64, 500000.0, sc), dtype=torch.float64).to(F32)
    assert rdim == 64 and not inter and torch.equal(inv.cpu(), want)
    part = POSITION_ENCODINGS.make("rope", head_dim=64, theta=10000.0, rotary_dim=32, interleaved=True)
    part.load({}, F32, torch.device(DEV))
    assert part.rotary_params()[1:] == (32, True) and part.rotary_params()[0].numel() == 16


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_swiglu_part(dtype):
    from photon_infer_amd.parts import FEED_FORWARDS
    D, I, T = 72, 200, 9
    W = {"gate_proj.weight": torch.randn(I, D, generator=gen(2)) * 0.2, "up_proj.weight": torch.randn(I, D, generator=gen(3)) * 0.2,
         "down_proj.weight": torch.randn(D, I, generator=gen(4)) * 0.2}
    ffn = load(FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=I), W, dtype)
    assert {s.name: s.shape for s in ffn.tensor_specs()} == {k: tuple(v.shape) for k, v in W.items()}
    h = torch.randn(T, D, generator=gen(5)).to(dtype)
    x0 = torch.randn(T, D, generator=gen(6))
    x = x0.clone().to(DEV)
    ffn.forward(h.to(DEV), x, None)          # no step context: no workspace, nothing is left pending
    Wr = {k: v.to(dtype).float() for k, v in W.items()}
    rd = (lambda t: t) if dtype == F32 else P.bf16_round
    act = rd(P.swiglu(rd(P.linear(h.float(), Wr["gate_proj.weight"])), rd(P.linear(h.float(), Wr["up_proj.weight"]))))
    want = x0 + P.linear(act, Wr["down_proj.weight"])
    assert (x.cpu() - want).abs().max() <= (2e-5 if dtype == F32 else 0.03)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("window", [None, 6])
def test_attention_part(dtype, window):
    """The mixer alone: projections, rotation, cache write, attention over pages, output
    projection into the residual - in two steps, so the second reads what the first wrote."""
    from photon_infer_amd import ops
    from photon_infer_amd.parts import MIXERS, POSITION_ENCODINGS, KVCacheSpec, LayerCache
    D, nh, nkv, hd, page = 80, 6, 2, 32, 4
    rope = POSITION_ENCODINGS.make("rope", head_dim=hd, theta=10000.0)
    W = {"q_proj.weight": torch.randn(nh * hd, D, generator=gen(7)) * 0.3, "k_proj.weight": torch.randn(nkv * hd, D, generator=gen(8)) * 0.3,
         "v_proj.weight": torch.randn(nkv * hd, D, generator=gen(9)) * 0.3, "o_proj.weight": torch.randn(D, nh * hd, generator=gen(10)) * 0.3}
    attn = load(MIXERS.make("attention", hidden_size=D, num_heads=nh, num_kv_heads=nkv, head_dim=hd, position=rope,
                            window=window), W, dtype)
    assert attn.cache_spec() == KVCacheSpec(nkv, hd, window)
    S, first = 23, 14
    h = torch.randn(S, D, generator=gen(11)).to(dtype)
    cache = LayerCache(group=0, k=torch.zeros(16, nkv, page, hd, dtype=dtype, device=DEV),
                       v=torch.zeros(16, nkv, hd, page, dtype=dtype, device=DEV), page_size=page)
    table = torch.tensor([[9, 2, 11, 5, 0, 7]], dtype=torch.int32, device=DEV)
    x = torch.zeros(S, D, device=DEV)
    for lo, hi in ((0, first), (first, S)):
        ctx = attention_ctx([hi - lo], [hi], dtype)
        ctx.block_tables = {0: table}
        xs = x[lo:hi]
        attn.forward(h[lo:hi].to(DEV), xs, ctx, cache)
    Wr = {k: v.to(dtype).float() for k, v in W.items()}
    rd = (lambda t: t) if dtype == F32 else P.bf16_round
    f = P.rope_frequencies(hd, 10000.0, None)
    q = rd(P.rope(rd(P.linear(h.float(), Wr["q_proj.weight"])).reshape(S, nh, hd), range(S), f, False))
    k = rd(P.rope(rd(P.linear(h.float(), Wr["k_proj.weight"])).reshape(S, nkv, hd), range(S), f, False))
    v = rd(P.linear(h.float(), Wr["v_proj.weight"])).reshape(S, nkv, hd)
    a = rd(P.attention(q, k, v, 1 / math.sqrt(hd), window=window).reshape(S, nh * hd))
    want = P.linear(a, Wr["o_proj.weight"])
    assert (x.cpu() - want).abs().max() <= (5e-5 if dtype == F32 else 0.02 * want.abs().max())


def test_tied_head_is_the_embedding_tensor(tmp_path):
    from photon_infer_amd.engine import EngineOptions, ModelRunner
    from tiny_models import make_model_dir
    tied = ModelRunner(make_model_dir(tmp_path, "A"), EngineOptions(dtype="bfloat16", block_size=4, num_blocks=8, max_batch=2))
    assert tied.model.head.weight.data_ptr() == tied.model.embedding.weight.data_ptr()
    untied = ModelRunner(make_model_dir(tmp_path, "B"), EngineOptions(dtype="bfloat16", block_size=8, num_blocks=8, max_batch=2))
    assert untied.model.head.weight.data_ptr() != untied.model.embedding.weight.data_ptr()


# ------------------------------------------------------------------ a toy architecture, defined here
def register_toy():
    """An architecture with a mixer that keeps a state of its own: the running sum of what it
    has seen of a request.  Layers alternate between it and attention; the run order names
    layer 0 twice and lets the last entry read the first attention layer's cache."""
    from photon_infer_amd import register_architecture
    from photon_infer_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, Mixer,
                                        ModelSpec, RunEntry, StateSpec, TokenEmbedding)
    from photon_infer_amd.weights import TensorSpec

    class RunningMean(Mixer):
        """out_t = W . mean(h_0 .. h_t).  State per request: [sum (D) | count (1)], float32."""

        def __init__(self, hidden_size):
            self.hidden_size = hidden_size

        def tensor_specs(self):
            return [TensorSpec("proj.weight", (self.hidden_size, self.hidden_size))]

        def cache_spec(self):
            return StateSpec((self.hidden_size + 1,), torch.float32)

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            self.w = tensors["proj.weight"].float()

        def forward(self, h, x, ctx, cache):
            start = 0
            for slot, n in zip(ctx.host_slots, ctx.q_lens):
                state = cache.state[slot]
                sums = state[:-1] + torch.cumsum(h[start:start + n].float(), 0)
                counts = state[-1] + torch.arange(1, n + 1, device=h.device, dtype=torch.float32)
                x[start:start + n] += (sums / counts[:, None]) @ self.w.t()
                state[:-1] = sums[-1]
                state[-1] = counts[-1]
                start += n

    MIXERS.register("running_mean", RunningMean)

    @dataclasses.dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        hidden_size: int
        vocab_size: int
        num_heads: int
        eps: float
        torch_dtype: str = "float32"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(raw["architectures"][0], raw["hidden_size"], raw["vocab_size"], raw["num_heads"], raw["eps"],
                       raw.get("torch_dtype", "float32"))

        def to_dict(self):
            d = dataclasses.asdict(self)
            d["architectures"] = [d.pop("architecture")]
            return d

    def build(cfg):
        D, hd = cfg.hidden_size, cfg.hidden_size // cfg.num_heads
        rope = POSITION_ENCODINGS.make("rope", head_dim=hd, theta=100.0)

        def block(mixer_prefix, mixer):
            return BLOCKS.make("prenorm", norm1=("n1.", NORMS.make("rmsnorm", dim=D, eps=cfg.eps)), mixer=(mixer_prefix, mixer),
                               norm2=("n2.", NORMS.make("rmsnorm", dim=D, eps=cfg.eps)),
                               ffn=("ffn.", FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=2 * D)))

        def attn(own_kv=True):
            return MIXERS.make("attention", hidden_size=D, num_heads=cfg.num_heads, num_kv_heads=1, head_dim=hd,
                               position=rope, own_kv=own_kv)
        layers = [("l0.", block("mean.", MIXERS.make("running_mean", hidden_size=D))), ("l1.", block("attn.", attn())),
                  ("l2.", block("attn.", attn(own_kv=False)))]
        order = [RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(2, cache_of=1)]
        return ModelSpec(hidden_size=D, vocab_size=cfg.vocab_size, max_positions=64,
                         embedding=("emb.", TokenEmbedding(cfg.vocab_size, D)), layers=layers, run_order=order,
                         final_norm=("norm.", NORMS.make("rmsnorm", dim=D, eps=cfg.eps)),
                         head=("head.", LMHead(cfg.vocab_size, D, tied=False)))

    register_architecture("ToyForCausalLM", ToyConfig, build)
    return ToyConfig


def plain_toy(cfg, W, toks):
    """The toy architecture on a whole sequence, from its definition."""
    D, nh = cfg["hidden_size"], cfg["num_heads"]
    hd, S, eps = D // nh, len(toks), cfg["eps"]
    f = P.rope_frequencies(hd, 100.0, None)
    x = P.embedding(W["emb.weight"], toks)

    def ffn(x, p):
        h = P.rmsnorm(x, W[p + "n2.weight"], eps)
        return x + P.linear(P.swiglu(P.linear(h, W[p + "ffn.gate_proj.weight"]), P.linear(h, W[p + "ffn.up_proj.weight"])),
                            W[p + "ffn.down_proj.weight"])

    def mean_layer(x):
        h = P.rmsnorm(x, W["l0.n1.weight"], eps)
        run = torch.cumsum(h, 0) / torch.arange(1, S + 1)[:, None]
        return ffn(x + P.linear(run, W["l0.mean.proj.weight"]), "l0.")

    x = mean_layer(x)
    h = P.rmsnorm(x, W["l1.n1.weight"], eps)
    q = P.rope(P.linear(h, W["l1.attn.q_proj.weight"]).reshape(S, nh, hd), range(S), f, False)
    k = P.rope(P.linear(h, W["l1.attn.k_proj.weight"]).reshape(S, 1, hd), range(S), f, False)
    v = P.linear(h, W["l1.attn.v_proj.weight"]).reshape(S, 1, hd)
    x = ffn(x + P.linear(P.attention(q, k, v, 1 / math.sqrt(hd)).reshape(S, D), W["l1.attn.o_proj.weight"]), "l1.")
    x = mean_layer(x)                                   # layer 0 again, with a state of its own
    h = P.rmsnorm(x, W["l2.n1.weight"], eps)            # reads layer 1's keys and values
    q2 = P.rope(P.linear(h, W["l2.attn.q_proj.weight"]).reshape(S, nh, hd), range(S), f, False)
    x = ffn(x + P.linear(P.attention(q2, k, v, 1 / math.sqrt(hd)).reshape(S, D), W["l2.attn.o_proj.weight"]), "l2.")
    return P.linear(P.rmsnorm(x, W["norm.weight"], eps), W["head.weight"])


def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    from photon_infer_amd import write_random_model
    from photon_infer_amd.engine import EngineOptions, ModelRunner, StepEntry
    ToyConfig = register_toy()
    cfg = ToyConfig("ToyForCausalLM", hidden_size=48, vocab_size=97, num_heads=3, eps=1e-5)
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=2, std=0.15, norm_init="uniform", dtype="float32")
    raw, W = P.read_model_folder(d)
    runner = ModelRunner(d, EngineOptions(dtype="float32", block_size=4, num_blocks=24, max_batch=2))
    # the plan: one page group (layer 1's; the last entry shares it), two state slabs (layer 0 runs twice)
    assert len(runner.plan.groups) == 1 and runner.plan.groups[0].owners == ((1, 0),)
    assert sorted(e for e, _ in runner.plan.states) == [(0, 0), (2, 0)]
    assert runner.layer_caches[3].k is runner.layer_caches[1].k and not runner.layer_caches[3].writes
    assert runner.layer_caches[0].state is not runner.layer_caches[2].state
    assert runner.states.bytes_per_slot == 2 * 49 * 4
    seqs = {"a": random_tokens(30, 97, 1), "b": random_tokens(21, 97, 2), "c": random_tokens(17, 97, 3)}
    want = {k: plain_toy(raw, W, v) for k, v in seqs.items()}

    def feed(rid, cuts):
        rows, i = [], 0
        for n in cuts:
            rows.append(runner.step([StepEntry(rid, seqs[rid][i:i + n], list(range(n)))]).cpu())
            i += n
        return torch.cat(rows)

    runner.admit("a")
    got = feed("a", [30])
    assert (got - want["a"]).abs().max() < 3e-5 * want["a"].abs().max().clamp(min=1)
    runner.release("a")
    # portions, two requests interleaved; "b" takes the slot "a" left, whose state must be cleared
    runner.admit("b"); runner.admit("c")
    out = {"b": [], "c": []}
    pos = {"b": 0, "c": 0}
    for nb, nc in [(5, 1), (1, 7), (2, 2), (13, 1), (0, 6)]:
        entries = [StepEntry(r, seqs[r][pos[r]:pos[r] + n], list(range(n))) for r, n in (("b", nb), ("c", nc)) if n]
        logits = runner.step(entries).cpu()
        i = 0
        for e in entries:
            out[e.rid].append(logits[i:i + len(e.tokens)]); i += len(e.tokens); pos[e.rid] += len(e.tokens)
    for r in ("b", "c"):
        got = torch.cat(out[r])
        assert got.shape == want[r].shape
        assert (got - want[r]).abs().max() < 3e-5 * want[r].abs().max().clamp(min=1), r


def test_toy_mixer_with_state_generates_through_the_engine(tmp_path):
    """The toy's mixer reads the requests' slots on the host, so it does not promise that its
    launches repeat (``graph_safe`` stays False): the engine with its default options (graphs,
    a step ahead) must notice and step it eagerly.  More requests than slots, so that slots and
    their state rows are used again; some greedy, some sampled."""
    from photon_infer_amd import ContinuousBatchEngine, write_random_model
    from photon_infer_amd.sampling import uniform_draw
    ToyConfig = register_toy()
    cfg = ToyConfig("ToyForCausalLM", hidden_size=48, vocab_size=97, num_heads=3, eps=1e-5)
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=3, std=0.15, norm_init="uniform", dtype="float32")
    raw, W = P.read_model_folder(d)
    eng = ContinuousBatchEngine(d, dtype="float32", block_size=4, num_blocks=48, max_batch=2, chunk_size=5)
    assert eng.options.use_graphs and eng.options.lookahead
    assert not eng.runner.graph_safe
    prompts = [random_tokens(n, 97, 10 + n) for n in (7, 3, 12, 5, 9)]
    new = [6, 11, 4, 9, 7]
    temps = [0.0, 0.8, 0.0, 0.0, 1.3]
    ids = [eng.add_request(p, n, temperature=t, seed=100 + i, ignore_eos=True) for i, (p, n, t) in enumerate(zip(prompts, new, temps))]
    eng.run_until_complete()
    assert not eng.runner._graphs                      # nothing was captured
    assert eng.runner.cache.num_live == 0
    for i, rid in enumerate(ids):
        got = eng.get_result(rid)
        assert len(got) == new[i]
        seq = list(prompts[i])
        for k, tok in enumerate(got):
            logits = plain_toy(raw, W, seq)[-1]
            if temps[i] == 0.0:
                assert logits[tok].item() >= logits.max().item() - 1e-4, (i, k)
            else:
                assert tok == P.sample_temperature(logits, temps[i], uniform_draw(100 + i, k)), (i, k)
            seq.append(tok)
    # the Llama parts all make the promise
    from tiny_models import make_model_dir
    llama = ContinuousBatchEngine(make_model_dir(tmp_path, "A"), dtype="float32", block_size=4, num_blocks=16, max_batch=2)
    assert llama.runner.graph_safe


# ------------------------------------------------------------------ a second toy: routing and another position scheme
def register_routed_toy():
    """A feed-forward that routes every token to one of several small experts (router logits in
    float32, the largest wins, lowest index among equals), and a position encoding that is no
    rotation: a learned table added to queries and keys.  Both defined here, registered by name,
    and chosen layer by layer: layer 0 routes, layer 1 has the ordinary gated feed-forward."""
    from photon_infer_amd import register_architecture
    from photon_infer_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, FeedForward, LMHead,
                                        ModelSpec, PositionEncoding, RunEntry, TokenEmbedding)
    from photon_infer_amd.weights import TensorSpec

    class RoutedExperts(FeedForward):
        def __init__(self, hidden_size, expert_size, num_experts, output_scale):
            self.D, self.I, self.E, self.scale = hidden_size, expert_size, num_experts, output_scale

        def tensor_specs(self):
            specs = [TensorSpec("router.weight", (self.E, self.D))]
            for e in range(self.E):
                specs += [TensorSpec(f"experts.{e}.up.weight", (self.I, self.D)), TensorSpec(f"experts.{e}.down.weight", (self.D, self.I))]
            return specs

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            self.router = tensors["router.weight"].float()
            self.up = [tensors[f"experts.{e}.up.weight"].float() for e in range(self.E)]
            self.down = [tensors[f"experts.{e}.down.weight"].float() for e in range(self.E)]

        def forward(self, h, x, ctx):
            hf = h.float()
            choice = (hf @ self.router.t()).argmax(dim=-1)          # float32 logits; argmax takes the lowest index among equals
            for e in range(self.E):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    x[rows] += self.scale * (torch.relu(hf[rows] @ self.up[e].t()) @ self.down[e].t())

    FEED_FORWARDS.register("routed_experts", RoutedExperts)

    class AddedPositions(PositionEncoding):
        """q and k of the token at position p get table[p] added, the same vector for every head."""

        def __init__(self, head_dim, max_positions):
            self.head_dim, self.max_positions = head_dim, max_positions

        def tensor_specs(self):
            return [TensorSpec("table", (self.max_positions, self.head_dim))]

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            self.table = tensors["table"].float()

        def apply(self, q, k, ctx):
            add = self.table[ctx.positions.long()]                  # [T, head_dim]
            for t in (q, k):
                if t is not None:
                    v = t.view(t.shape[0], -1, self.head_dim)
                    v += add[:, None, :].to(t.dtype)

    POSITION_ENCODINGS.register("added_positions", AddedPositions)

    @dataclasses.dataclass(frozen=True)
    class RoutedConfig:
        architecture: str
        width: int
        vocab: int
        heads: int
        experts: int
        expert_width: int
        expert_scale: float
        norm_eps: float
        torch_dtype: str = "float32"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(raw["architectures"][0], raw["width"], raw["vocab"], raw["heads"], raw["experts"], raw["expert_width"],
                       raw["expert_scale"], raw["norm_eps"], raw.get("torch_dtype", "float32"))

        def to_dict(self):
            d = dataclasses.asdict(self)
            d["architectures"] = [d.pop("architecture")]
            return d

    def build(cfg):
        D, hd = cfg.width, cfg.width // cfg.heads
        norm = lambda: NORMS.make("rmsnorm", dim=D, eps=cfg.norm_eps)

        def block(ffn):
            # every layer has a position table of its own: the part is given under the mixer's prefix
            mixer = MIXERS.make("attention", hidden_size=D, num_heads=cfg.heads, num_kv_heads=cfg.heads, head_dim=hd,
                                position=POSITION_ENCODINGS.make("added_positions", head_dim=hd, max_positions=40))
            return BLOCKS.make("prenorm", norm1=("n1.", norm()), mixer=("attn.", mixer), norm2=("n2.", norm()), ffn=("ffn.", ffn))
        layers = [("l0.", block(FEED_FORWARDS.make("routed_experts", hidden_size=D, expert_size=cfg.expert_width,
                                                    num_experts=cfg.experts, output_scale=cfg.expert_scale))),
                  ("l1.", block(FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=3 * D)))]
        return ModelSpec(hidden_size=D, vocab_size=cfg.vocab, max_positions=40, embedding=("emb.", TokenEmbedding(cfg.vocab, D)),
                         layers=layers, run_order=[RunEntry(0), RunEntry(1)], final_norm=("norm.", norm()),
                         head=("head.", LMHead(cfg.vocab, D, tied=True)))

    register_architecture("RoutedToyForCausalLM", RoutedConfig, build)
    return RoutedConfig


def plain_routed_toy(cfg, W, toks):
    D, nh, S, eps = cfg["width"], cfg["heads"], len(toks), cfg["norm_eps"]
    hd = D // nh
    x = P.embedding(W["emb.weight"], toks)
    for l in ("l0.", "l1."):
        h = P.rmsnorm(x, W[l + "n1.weight"], eps)
        add = W[l + "attn.position.table"][:S][:, None, :]
        q = P.linear(h, W[l + "attn.q_proj.weight"]).reshape(S, nh, hd) + add
        k = P.linear(h, W[l + "attn.k_proj.weight"]).reshape(S, nh, hd) + add
        v = P.linear(h, W[l + "attn.v_proj.weight"]).reshape(S, nh, hd)
        x = x + P.linear(P.attention(q, k, v, 1 / math.sqrt(hd)).reshape(S, D), W[l + "attn.o_proj.weight"])
        h = P.rmsnorm(x, W[l + "n2.weight"], eps)
        if l == "l0.":
            choice = P.linear(h, W[l + "ffn.router.weight"]).argmax(dim=-1)
            out = torch.zeros_like(x)
            for t in range(S):
                e = int(choice[t])
                out[t] = cfg["expert_scale"] * P.linear(torch.relu(P.linear(h[t:t + 1], W[f"{l}ffn.experts.{e}.up.weight"])),
                                                         W[f"{l}ffn.experts.{e}.down.weight"])[0]
            x = x + out
        else:
            x = x + P.linear(P.swiglu(P.linear(h, W[l + "ffn.gate_proj.weight"]), P.linear(h, W[l + "ffn.up_proj.weight"])),
                             W[l + "ffn.down_proj.weight"])
    return P.linear(P.rmsnorm(x, W["norm.weight"], eps), W["emb.weight"]), None


def test_toy_routed_feed_forward_and_added_positions(tmp_path):
    """Registered from here: a feed-forward with routing and a position encoding that is not a
    rotation; built from config.json, stepped whole and in portions beside another request."""
    from photon_infer_amd import write_random_model
    from photon_infer_amd.engine import EngineOptions, ModelRunner, StepEntry
    RoutedConfig = register_routed_toy()
    cfg = RoutedConfig("RoutedToyForCausalLM", width=32, vocab=83, heads=2, experts=3, expert_width=56, expert_scale=0.7, norm_eps=1e-6)
    d = write_random_model(cfg, str(tmp_path / "routed"), seed=5, std=0.2, norm_init="uniform", dtype="float32")
    raw, W = P.read_model_folder(d)
    assert "l0.attn.position.table" in W and "l1.attn.position.table" in W and "l0.ffn.experts.2.down.weight" in W
    runner = ModelRunner(d, EngineOptions(dtype="float32", block_size=4, num_blocks=20, max_batch=2))
    seqs = {"a": random_tokens(26, 83, 4), "b": random_tokens(19, 83, 5)}
    want = {k: plain_routed_toy(raw, W, v)[0] for k, v in seqs.items()}
    runner.admit("a")
    got = runner.step([StepEntry("a", seqs["a"], list(range(26)))]).cpu()
    assert (got - want["a"]).abs().max() < 3e-5 * want["a"].abs().max().clamp(min=1)
    runner.release("a")
    runner.admit("a"); runner.admit("b")
    out, pos = {"a": [], "b": []}, {"a": 0, "b": 0}
    for na, nb in [(3, 2), (1, 9), (12, 1), (10, 1), (0, 6)]:
        entries = [StepEntry(r, seqs[r][pos[r]:pos[r] + n], list(range(n))) for r, n in (("a", na), ("b", nb)) if n]
        logits = runner.step(entries).cpu()
        i = 0
        for e in entries:
            out[e.rid].append(logits[i:i + len(e.tokens)]); i += len(e.tokens); pos[e.rid] += len(e.tokens)
    for r in ("a", "b"):
        got = torch.cat(out[r])
        assert got.shape == want[r].shape
        assert (got - want[r]).abs().max() < 3e-5 * want[r].abs().max().clamp(min=1), r
