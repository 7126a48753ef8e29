"""The seams for other architectures, exercised by toy parts that this file defines and registers
without touching the framework:

* another arrangement of a block (norm once, mixer and feed-forward side by side, the norm read
  through a library call), between ordinary pre-norm blocks, at sizes where the ordinary blocks
  leave their updates of the stream in pieces - the new arrangement must never meet a stale stream;
* a block with two mixers side by side, one of which pages a single latent vector per token (its
  own tensor, shape and dtype) next to attention's keys and values, stepped under every cutting
  and generated with through the engine.
"""
import dataclasses
import math

import pytest
import torch

import plain_llama as P
import plain_wide as PW
from tiny_models import random_tokens

pytestmark = pytest.mark.gpu


@dataclasses.dataclass(frozen=True)
class SeamConfig:
    architecture: str
    hidden_size: int
    intermediate_size: int
    vocab_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    eps: float
    latent: int = 0
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        fields = {f.name for f in dataclasses.fields(cls)} - {"architecture"}
        return cls(raw["architectures"][0], **{k: v for k, v in raw.items() if k in fields})

    def to_dict(self):
        d = dataclasses.asdict(self)
        d["architectures"] = [d.pop("architecture")]
        return d


def _llama_parts(cfg):
    from photon_infer_amd.parts import FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS
    rope = POSITION_ENCODINGS.make("rope", head_dim=cfg.head_dim, theta=10000.0)

    def norm():
        return NORMS.make("rmsnorm", dim=cfg.hidden_size, eps=cfg.eps)

    def attn():
        return MIXERS.make("attention", hidden_size=cfg.hidden_size, num_heads=cfg.num_heads, num_kv_heads=cfg.num_kv_heads,
                           head_dim=cfg.head_dim, position=rope)

    def ffn():
        return FEED_FORWARDS.make("swiglu", hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size)

    return norm, attn, ffn


# ------------------------------------------------------------------ plain forms of the shared pieces
def _plain_attn(cfg, W, p, h, rd):
    S, nh, nkv, hd = h.shape[0], cfg["num_heads"], cfg["num_kv_heads"], cfg["head_dim"]
    f = P.rope_frequencies(hd, 10000.0, None)
    pos = torch.arange(S)
    q = rd(PW.rope(rd(h @ W[p + "q_proj.weight"].t()).reshape(S, nh, hd), pos, f, False))
    k = rd(PW.rope(rd(h @ W[p + "k_proj.weight"].t()).reshape(S, nkv, hd), pos, f, False))
    v = rd(h @ W[p + "v_proj.weight"].t()).reshape(S, nkv, hd)
    a = rd(PW.attention(q, k, v, 1 / math.sqrt(hd), None, rd if rd is not _same else None).reshape(S, nh * hd))
    return a @ W[p + "o_proj.weight"].t()


def _plain_ffn(W, p, h, rd):
    return rd(P.swiglu(rd(h @ W[p + "gate_proj.weight"].t()), rd(h @ W[p + "up_proj.weight"].t()))) @ W[p + "down_proj.weight"].t()


def _same(t):
    return t


def _plain_prenorm(cfg, W, p, x, rd):
    x = x + _plain_attn(cfg, W, p + "attn.", rd(PW.rmsnorm(x, W[p + "n1.weight"], cfg["eps"])), rd)
    return x + _plain_ffn(W, p + "ffn.", rd(PW.rmsnorm(x, W[p + "n2.weight"], cfg["eps"])), rd)


# ------------------------------------------------------------------ another arrangement
def register_parallel():
    """``x += mixer(n(x)) + ffn(n(x))`` with one norm that reads the stream through torch, as the
    middle layer of three; the outer two are the ordinary pre-norm blocks."""
    from photon_infer_amd import register_architecture
    from photon_infer_amd.parts import BLOCKS, NORMS, Block, LMHead, ModelSpec, Norm, TokenEmbedding
    from photon_infer_amd.weights import TensorSpec

    class TorchRMSNorm(Norm):
        """Reads the stream with library calls: it knows nothing of updates left in pieces."""

        def __init__(self, dim, eps):
            self.dim, self.eps = dim, eps

        def tensor_specs(self):
            return [TensorSpec("weight", (self.dim,), "norm")]

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            self.weight = tensors["weight"].float()

        def forward(self, x, ctx=None, rows=None):
            x = x if rows is None else x[rows.long()]
            rms = torch.sqrt((x * x).sum(-1, keepdim=True) / self.dim + self.eps)
            return (self.weight * (x * (1.0 / rms))).to(self.dtype)

    NORMS.register("torch_rmsnorm", TorchRMSNorm)

    class ParallelBlock(Block):
        """Knows nothing of deferred updates: sets no flag, calls no ``materialize``."""

        def __init__(self, norm, mixer, ffn):
            self._named = [norm, mixer, ffn]
            self.norm, self.mixer, self.ffn = norm[1], mixer[1], ffn[1]

        def tensor_specs(self):
            return [s.with_prefix(p) for p, part in self._named for s in part.tensor_specs()]

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            for prefix, part in self._named:
                part.load({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, dtype, device)

        def forward(self, x, ctx, cache):
            h = self.norm.forward(x, ctx)
            self.mixer.forward(h, x, ctx, cache)
            self.ffn.forward(h, x, ctx)

    BLOCKS.register("parallel", ParallelBlock)

    def build(cfg):
        norm, attn, ffn = _llama_parts(cfg)
        D = cfg.hidden_size

        def prenorm():
            return BLOCKS.make("prenorm", norm1=("n1.", norm()), mixer=("attn.", attn()), norm2=("n2.", norm()), ffn=("ffn.", ffn()))

        layers = [("l0.", prenorm()),
                  ("l1.", BLOCKS.make("parallel", norm=("n.", NORMS.make("torch_rmsnorm", dim=D, eps=cfg.eps)),
                                      mixer=("attn.", attn()), ffn=("ffn.", ffn()))),
                  ("l2.", prenorm())]
        return ModelSpec(hidden_size=D, vocab_size=cfg.vocab_size, max_positions=1024,
                         embedding=("emb.", TokenEmbedding(cfg.vocab_size, D)), layers=layers,
                         final_norm=("norm.", NORMS.make("torch_rmsnorm", dim=D, eps=cfg.eps)),
                         head=("head.", LMHead(cfg.vocab_size, D, tied=True)))

    register_architecture("ParallelToyForCausalLM", SeamConfig, build)


def plain_parallel(cfg, W, toks, rd=_same):
    W = {k: v.float() for k, v in W.items()}
    x = W["emb.weight"][torch.tensor(toks)]
    x = _plain_prenorm(cfg, W, "l0.", x, rd)
    h = rd(PW.rmsnorm(x, W["l1.n.weight"], cfg["eps"]))
    x = x + _plain_attn(cfg, W, "l1.attn.", h, rd) + _plain_ffn(W, "l1.ffn.", h, rd)
    x = _plain_prenorm(cfg, W, "l2.", x, rd)
    return rd(PW.rmsnorm(x, W["norm.weight"], cfg["eps"])) @ W["emb.weight"].t()


def test_another_arrangement_never_meets_a_stream_in_pieces(tmp_path):
    """Hidden 1,024 and intermediate 2,816 (the sizes at which the o and down projections are cut
    over k and left in pieces for the next norm), bfloat16: a whole prompt of 150 tokens (tile
    kernels), portions of 40 and 7, then single tokens (weight-streaming kernels).  The pre-norm
    blocks do defer (the counters say so); the parallel block and the library-call norms read the
    finished stream, so the logits are the plain form's."""
    from photon_infer_amd import write_random_model
    from photon_infer_amd.engine import EngineOptions, ModelRunner, StepEntry
    register_parallel()
    cfg = SeamConfig("ParallelToyForCausalLM", hidden_size=1024, intermediate_size=2816, vocab_size=4096, num_heads=16,
                     num_kv_heads=4, head_dim=64, eps=1e-5)
    d = write_random_model(cfg, str(tmp_path / "par"), seed=4, std=0.03, norm_init="uniform", dtype="bfloat16")
    raw, W = P.read_model_folder(d)
    runner = ModelRunner(d, EngineOptions(dtype="bfloat16", block_size=16, num_blocks=64, max_batch=2))
    assert not runner.graph_safe                      # the library-call norm makes no promise
    toks = random_tokens(150 + 40 + 7 + 12, 4096, 9)
    ref = plain_parallel(raw, W, toks)
    emu = plain_parallel(raw, W, toks, P.bf16_round)
    tol = 3.0 * (emu - ref).abs().max().item()
    runner.admit("a")
    rows, i = [], 0
    for n in [150, 40, 7] + [1] * 12:
        rows.append(runner.step([StepEntry("a", toks[i:i + n], list(range(n)))]).cpu())
        i += n
    got = torch.cat(rows)
    counts = runner.workspace.counts
    assert counts["deferred"] > 0 and counts["added_by_norm"] > 0, counts       # the pre-norm blocks did leave pieces
    assert counts["added_by_norm"] + counts["applied"] + counts["flushed"] == counts["deferred"], counts   # and every one was added once
    err = (got - ref).abs().max().item()
    assert err <= tol, (err, tol)
    assert tol < 0.1 * ref.abs().max().item()


# ------------------------------------------------------------------ two mixers in a block, one paging a latent
def register_two_mixers():
    from photon_infer_amd import register_architecture
    from photon_infer_amd.parts import (BLOCKS, MIXERS, NORMS, PAGE, Block, LMHead, Mixer, ModelSpec, PagedCacheSpec, PagedTensor,
                                        TokenEmbedding)
    from photon_infer_amd.weights import TensorSpec

    class LatentMean(Mixer):
        """Keeps one latent vector per token, ``z_t = W_in h_t`` (float32, width L), in pages of its
        own tensor, and adds ``W_out mean(z_0 .. z_t)`` to the stream.  Everything by library
        calls on the host's view of the step, so it promises no graph."""

        def __init__(self, hidden_size, latent):
            self.D, self.L = hidden_size, latent

        def tensor_specs(self):
            return [TensorSpec("in.weight", (self.L, self.D)), TensorSpec("out.weight", (self.D, self.L))]

        def cache_spec(self):
            return PagedCacheSpec((PagedTensor("latent", (PAGE, self.L), torch.float32),))

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            self.w_in, self.w_out = tensors["in.weight"].float(), tensors["out.weight"].float()

        def forward(self, h, x, ctx, cache):
            pool = cache.tensors["latent"]                     # [pages, page, L]
            flat = pool.view(-1, self.L)
            table = ctx.block_tables[cache.group]
            z = h.float() @ self.w_in.t()
            start = 0
            for r, (n, kv) in enumerate(zip(ctx.q_lens, ctx.kv_lens)):
                pos = torch.arange(kv, device=h.device)
                where = table[r].long()[pos // cache.page_size] * cache.page_size + pos % cache.page_size
                flat[where[kv - n:]] = z[start:start + n]      # this step's tokens
                seen = flat[where]                             # every token of the request so far, from its pages
                means = torch.cumsum(seen, 0)[kv - n:] / torch.arange(kv - n + 1, kv + 1, device=h.device)[:, None]
                x[start:start + n] += means @ self.w_out.t()
                start += n

    MIXERS.register("latent_mean", LatentMean)

    class TwoMixerBlock(Block):
        """``x += attention(n1(x)) + latent(n1(x)); x += ffn(n2(x))``."""

        def __init__(self, norm1, attn, latent, norm2, ffn):
            self._named = [norm1, attn, latent, norm2, ffn]
            self.norm1, self.attn, self.latent, self.norm2, self.ffn = (p[1] for p in self._named)

        def mixers(self):
            return [self.attn, self.latent]

        def tensor_specs(self):
            return [s.with_prefix(p) for p, part in self._named for s in part.tensor_specs()]

        def load(self, tensors, dtype, device):
            super().load(tensors, dtype, device)
            for prefix, part in self._named:
                part.load({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, dtype, device)

        def forward(self, x, ctx, caches):
            h = self.norm1.forward(x, ctx)
            self.attn.forward(h, x, ctx, caches[0])
            self.latent.forward(h, x, ctx, caches[1])
            self.ffn.forward(self.norm2.forward(x, ctx), x, ctx)

    BLOCKS.register("two_mixers", TwoMixerBlock)

    def build(cfg):
        norm, attn, ffn = _llama_parts(cfg)
        D = cfg.hidden_size
        layers = [(f"l{i}.", BLOCKS.make("two_mixers", norm1=("n1.", norm()), attn=("attn.", attn()),
                                         latent=("lat.", MIXERS.make("latent_mean", hidden_size=D, latent=cfg.latent)),
                                         norm2=("n2.", norm()), ffn=("ffn.", ffn()))) for i in range(2)]
        return ModelSpec(hidden_size=D, vocab_size=cfg.vocab_size, max_positions=256,
                         embedding=("emb.", TokenEmbedding(cfg.vocab_size, D)), layers=layers,
                         final_norm=("norm.", norm()), head=("head.", LMHead(cfg.vocab_size, D, tied=False)))

    register_architecture("TwoMixerToyForCausalLM", SeamConfig, build)


def plain_two_mixers(cfg, W, toks):
    W = {k: v.float() for k, v in W.items()}
    S = len(toks)
    x = W["emb.weight"][torch.tensor(toks)]
    for i in range(2):
        p = f"l{i}."
        h = PW.rmsnorm(x, W[p + "n1.weight"], cfg["eps"])
        z = h @ W[p + "lat.in.weight"].t()
        means = torch.cumsum(z, 0) / torch.arange(1, S + 1)[:, None]
        x = x + _plain_attn(cfg, W, p + "attn.", h, _same) + means @ W[p + "lat.out.weight"].t()
        x = x + _plain_ffn(W, p + "ffn.", PW.rmsnorm(x, W[p + "n2.weight"], cfg["eps"]), _same)
    return PW.rmsnorm(x, W["norm.weight"], cfg["eps"]) @ W["head.weight"].t()


def _two_mixer_model(tmp_path):
    from photon_infer_amd import write_random_model
    register_two_mixers()
    cfg = SeamConfig("TwoMixerToyForCausalLM", hidden_size=80, intermediate_size=136, vocab_size=211, num_heads=4,
                     num_kv_heads=2, head_dim=16, eps=1e-5, latent=24, torch_dtype="float32")
    d = write_random_model(cfg, str(tmp_path / "two"), seed=6, std=0.12, norm_init="uniform", dtype="float32")
    return d, P.read_model_folder(d)


def test_two_mixers_in_a_block_one_paging_a_latent_vector(tmp_path):
    """The cache follows each mixer's own description: per layer keys and values of attention
    and, beside them, the latent mixer's single float32 tensor; both mixers of a block share the
    request's block table.  Whole, in portions, and two requests mixed, with pages used again."""
    from photon_infer_amd.engine import EngineOptions, ModelRunner, StepEntry
    d, (raw, W) = _two_mixer_model(tmp_path)
    runner = ModelRunner(d, EngineOptions(dtype="float32", block_size=8, num_blocks=12, max_batch=2))
    plan = runner.plan
    assert len(plan.groups) == 1 and plan.groups[0].owners == ((0, 0), (0, 1), (1, 0), (1, 1))
    assert [[t.name for t in owner] for owner in plan.groups[0].tensors] == [["k", "v"], ["latent"]] * 2
    attn_view, latent_view = runner.layer_caches[0]
    assert attn_view.k.shape == (12, 2, 8, 16) and attn_view.v.shape == (12, 2, 16, 8)
    assert latent_view.tensors["latent"].shape == (12, 8, 24) and latent_view.tensors["latent"].dtype == torch.float32
    assert latent_view.k is None and attn_view.group == latent_view.group == 0
    seqs = {"a": random_tokens(50, 211, 1), "b": random_tokens(37, 211, 2), "c": random_tokens(29, 211, 3)}
    want = {k: plain_two_mixers(raw, W, v) for k, v in seqs.items()}

    def close(got, ref):
        return (got - ref).abs().max() < 5e-5 * ref.abs().max().clamp(min=1)

    runner.admit("a")
    assert close(runner.step([StepEntry("a", seqs["a"], list(range(50)))]).cpu(), want["a"])
    runner.release("a")                                   # its pages go back and are taken again below
    runner.admit("b"); runner.admit("c")
    out, pos = {"b": [], "c": []}, {"b": 0, "c": 0}
    for nb, nc in [(9, 1), (1, 6), (2, 2), (17, 1), (8, 19)]:
        entries = [StepEntry(r, seqs[r][pos[r]:pos[r] + n], list(range(n))) for r, n in (("b", nb), ("c", nc)) if n]
        logits = runner.step(entries).cpu()
        i = 0
        for e in entries:
            out[e.rid].append(logits[i:i + len(e.tokens)]); i += len(e.tokens); pos[e.rid] += len(e.tokens)
    for r in ("b", "c"):
        assert close(torch.cat(out[r]), want[r]), r
    runner.release("b"); runner.release("c")
    assert runner.cache.free_pages() == 12
    runner.cache.check_invariants()


def test_two_mixers_generate_through_the_engine(tmp_path):
    from photon_infer_amd import ContinuousBatchEngine
    d, (raw, W) = _two_mixer_model(tmp_path)
    eng = ContinuousBatchEngine(d, dtype="float32", block_size=8, num_blocks=24, max_batch=2, chunk_size=6)
    assert not eng.runner.graph_safe
    prompts = [random_tokens(n, 211, 20 + n) for n in (9, 4, 15)]
    outs = eng.generate(prompts, max_new_tokens=8, ignore_eos=True)
    assert eng.runner.cache.num_live == 0 and eng.runner.cache.free_pages() == 24
    for p, out in zip(prompts, outs):
        seq = list(p)
        for tok in out:
            logits = plain_two_mixers(raw, W, seq)[-1]
            assert logits[tok].item() >= logits.max().item() - 1e-4
            seq.append(tok)
