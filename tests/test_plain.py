"""Pins the plain implementation by what fixes it beside the reference's text (CPU):
the vectors the reference's own tests hold, special cases that reduce to a library
routine, and invariants - each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

import plain_llama as P
from tiny_models import TINY_A, TINY_B


# ------------------------------------------------------------------ vectors of the reference's tests
def test_rmsnorm_vectors():
    # tests/ops/test_rmsnorm.cpp:102-181
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    y = P.rmsnorm(x, torch.ones(4), 1e-5)
    assert torch.allclose(y, x / math.sqrt(7.5 + 1e-5), atol=1e-6)
    x2 = torch.tensor([[2.0, 4.0, 6.0, 8.0]])
    w2 = torch.tensor([0.5, 1.0, 1.5, 2.0])
    assert torch.allclose(P.rmsnorm(x2, w2, 1e-5), w2 * x2 / math.sqrt(30 + 1e-5), atol=1e-6)
    # eps is inside the root (outside, eps = 1 would give x / (sqrt(7.5) + 1))
    assert torch.allclose(P.rmsnorm(x, torch.ones(4), 1.0), x / math.sqrt(8.5), atol=1e-6)
    # no mean-centring: a constant row is not sent to zero
    assert torch.allclose(P.rmsnorm(torch.full((1, 4), 3.0), torch.ones(4), 0.0), torch.ones(1, 4), atol=1e-6)


def test_rmsnorm_invariants():
    x = torch.randn(5, 24, generator=torch.Generator().manual_seed(0))
    y = P.rmsnorm(x, torch.ones(24), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5), atol=1e-5)
    assert torch.allclose(P.rmsnorm(7.0 * x, torch.ones(24), 0.0), y, atol=1e-5)
    assert torch.allclose(y, x / x.norm(dim=-1, keepdim=True) * math.sqrt(24), atol=1e-5)


def test_linear_vectors():
    # tests/ops/test_matmul.cpp:90-204: weights are [out, in], y = x W^T
    W = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    assert P.linear(torch.tensor([[1.0, 2.0, 3.0]]), W).tolist() == [[14.0, 32.0]]
    assert P.linear(torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]]), W).tolist() == [[14.0, 32.0], [32.0, 77.0]]


def test_swiglu_vectors():
    # tests/ops/test_swiglu.cpp:159-216
    g = torch.tensor([1.0, 2.0, 3.0, 4.0])
    u = torch.tensor([0.5, 1.0, 1.5, 2.0])
    want = torch.tensor([x / (1 + math.exp(-x)) * v for x, v in zip(g.tolist(), u.tolist())])
    assert torch.allclose(P.swiglu(g, u), want, atol=1e-6)
    assert torch.equal(P.swiglu(torch.zeros(4), u), torch.zeros(4))
    big = P.swiglu(torch.tensor([50.0, -50.0, -200.0]), torch.tensor([2.0, 2.0, 2.0]))
    assert torch.allclose(big, torch.tensor([100.0, 0.0, 0.0]), atol=1e-6) and not torch.isnan(big).any()
    # the gate, not the up projection, goes through the sigmoid
    assert not torch.allclose(P.swiglu(g, u), P.swiglu(u, g))


def test_attention_vectors():
    # tests/ops/test_mha.cpp:29-174: one head, position 0 -> the value itself
    q = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]])
    k = torch.tensor([[[1.0, 1.0, 1.0, 1.0]]])
    v = torch.tensor([[[2.0, 3.0, 4.0, 5.0]]])
    assert torch.allclose(P.attention(q, k, v, 0.5)[0, 0], v[0, 0])
    # two heads of size 2, position 1: scores [1/sqrt(2), 0] per head
    q = torch.tensor([[[0.0, 0.0], [0.0, 0.0]], [[1.0, 0.0], [1.0, 0.0]]])
    k = torch.tensor([[[1.0, 0.0], [1.0, 0.0]], [[0.0, 1.0], [0.0, 1.0]]])
    v = torch.tensor([[[2.0, 3.0], [6.0, 7.0]], [[4.0, 5.0], [8.0, 9.0]]])
    out = P.attention(q, k, v, 1.0 / math.sqrt(2.0))
    w = torch.softmax(torch.tensor([1.0 / math.sqrt(2.0), 0.0]), 0)
    assert torch.allclose(out[1, 0], w[0] * v[0, 0] + w[1] * v[1, 0], atol=1e-6)
    assert torch.allclose(out[1, 1], w[0] * v[0, 1] + w[1] * v[1, 1], atol=1e-6)


def test_argmax_and_sampling_vectors():
    # tests/model/test_llama_model.cpp:236-249
    l = torch.arange(10, dtype=torch.float32)
    l[7] = 100.0
    assert P.argmax(l) == 7
    assert P.argmax(torch.tensor([1.0, 5.0, 5.0, 2.0])) == 1            # the first of equals
    p = torch.softmax(torch.tensor([0.0, 1.0, 2.0]) / 0.8, 0)
    lg = torch.tensor([0.0, 1.0, 2.0])
    assert P.sample_temperature(lg, 0.8, float(p[0]) * 0.5) == 0
    assert P.sample_temperature(lg, 0.8, float(p[0]) + 1e-4) == 1
    assert P.sample_temperature(lg, 0.8, 0.9999999) == 2
    assert P.sample_temperature(lg, 1e-3, 0.5) == 2                     # T -> 0 is the argmax


# ------------------------------------------------------------------ rotation
def test_rope_reference_table_and_identity():
    # tests/ops/test_rope.cpp:54-76,125-193: sin[pos=1, j=0] = sin(1); position 0 is the identity
    f = P.rope_frequencies(8, 10000.0, None)
    assert f[0] == 1.0 and abs(f[1] - 10000.0 ** (-2 / 8)) < 1e-15
    x = torch.randn(1, 2, 8, generator=torch.Generator().manual_seed(1))
    assert torch.equal(P.rope(x, [0], f, True), x)
    y = P.rope(x, [1], f, True)
    assert torch.allclose(y[0, 0, 0], x[0, 0, 0] * math.cos(1.0) - x[0, 0, 1] * math.sin(1.0), atol=1e-6)
    assert torch.allclose(y[0, 0, 1], x[0, 0, 0] * math.sin(1.0) + x[0, 0, 1] * math.cos(1.0), atol=1e-6)
    # rotation keeps each pair's norm
    assert torch.allclose(y[..., 0::2] ** 2 + y[..., 1::2] ** 2, x[..., 0::2] ** 2 + x[..., 1::2] ** 2, atol=1e-5)


def test_rope_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(2)
    f = P.rope_frequencies(16, 500000.0, TINY_B["rope_scaling"])
    q, k = torch.randn(1, 1, 16, generator=g, dtype=torch.float64), torch.randn(1, 1, 16, generator=g, dtype=torch.float64)
    for inter in (False, True):
        def score(m, n):
            return (P.rope(q, [m], f, inter) * P.rope(k, [n], f, inter)).sum().item()
        assert abs(score(5, 2) - score(40, 37)) < 1e-5      # float32 angles limit this
        assert abs(score(5, 2) - score(2, 5)) > 1e-3        # a wrong sign would pass the line above only


def test_rope_pairings_agree_under_the_row_permutation():
    # half-split pairing on permuted rows equals interleaved pairing: x_half[j] = x_int[2j], x_half[j + h] = x_int[2j+1]
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 2, 8, generator=g)
    f = P.rope_frequencies(8, 10000.0, None)
    perm = torch.tensor([0, 2, 4, 6, 1, 3, 5, 7])
    a = P.rope(x, [3, 4, 9], f, True)
    b = P.rope(x[..., perm], [3, 4, 9], f, False)
    assert torch.allclose(a[..., perm], b, atol=1e-6)


def test_llama3_scaling_hits_all_three_regimes():
    sc = TINY_B["rope_scaling"]          # factor 8, low 1, high 4, L 64; head_dim 32
    base = P.rope_frequencies(32, 500000.0, None)
    f = P.rope_frequencies(32, 500000.0, sc)
    lam = [2 * math.pi / b for b in base]
    kept = [j for j in range(16) if lam[j] < 64 / 4]
    low = [j for j in range(16) if lam[j] > 64 / 1]
    mid = [j for j in range(16) if j not in kept and j not in low]
    assert kept and low and mid
    assert all(f[j] == base[j] for j in kept)
    assert all(abs(f[j] - base[j] / 8) < 1e-18 for j in low)
    assert all(base[j] / 8 < f[j] < base[j] for j in mid)
    assert all(f[j] > f[j + 1] for j in range(15))                      # monotone across both thresholds
    one = dict(sc, factor=1.0)
    assert all(abs(a - b) < 1e-15 for a, b in zip(P.rope_frequencies(32, 500000.0, one), base))
    lin = P.rope_frequencies(32, 500000.0, {"rope_type": "linear", "factor": 4.0})
    assert all(abs(a - b / 4) < 1e-18 for a, b in zip(lin, base))


def _both_frequency_tables(rotary_dim, theta, sc):
    """The plain implementation's frequencies and the product's, for the same constants."""
    from photon_infer_amd.config.llama import RopeScaling
    from photon_infer_amd.parts.rope import rope_frequencies

    plain = P.rope_frequencies(rotary_dim, theta, sc)
    typed = None if sc is None else RopeScaling(**sc)
    return (("plain", plain), ("product", rope_frequencies(rotary_dim, theta, typed).tolist()))


def test_llama3_blend_falls_from_one_to_one_over_factor():
    # head size 128 with the constants of the 1B model: six pairs lie in the blended band.  The
    # ratio scaled / base must fall with the pair index from 1 (short wavelengths are kept) to
    # 1 / factor.  A blend with its two weights exchanged rises inside the band instead.
    sc = dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=8192)
    base = P.rope_frequencies(128, 500000.0, None)
    lam = [2 * math.pi / b for b in base]
    mid = [j for j in range(64) if 8192 / 4 <= lam[j] <= 8192 / 1]
    assert len(mid) >= 5 and mid == list(range(mid[0], mid[-1] + 1))
    for who, f in _both_frequency_tables(128, 500000.0, sc):
        ratio = [a / b for a, b in zip(f, base)]
        assert all(abs(r - 1.0) < 1e-13 for r in ratio[:mid[0]]), who
        assert all(abs(r - 1 / 32) < 1e-13 for r in ratio[mid[-1] + 1:]), who
        assert all(ratio[j] > ratio[j + 1] for j in range(mid[0] - 1, mid[-1] + 1)), who
        assert all(1 / 32 < ratio[j] < 1.0 for j in mid), who
        # the band's formula: linear in L / wavelength between the two ends
        for j in mid:
            s = (8192 / lam[j] - 1.0) / (4.0 - 1.0)
            assert abs(ratio[j] - ((1 - s) / 32 + s)) < 1e-12, (who, j)


def test_llama3_blend_is_continuous_at_both_thresholds():
    # Move the original context length so that one pair's wavelength sits a hair inside the band at
    # its short end, then at its long end: the ratio there is (almost) 1 and (almost) 1 / factor.
    # Exchanged weights give 1 / factor and 1; a band test with "<" for "<=" is caught as well.
    base = P.rope_frequencies(64, 500000.0, None)
    j = 20
    lam = 2 * math.pi / base[j]
    for L, want in ((lam * 4.0 * (1 + 1e-9), 1.0), (lam * 1.0 * (1 - 1e-9), 1 / 16)):
        sc = dict(rope_type="llama3", factor=16.0, low_freq_factor=1.0, high_freq_factor=4.0,
                  original_max_position_embeddings=L)
        for who, f in _both_frequency_tables(64, 500000.0, sc):
            assert abs(f[j] / base[j] - want) < 1e-7, (who, L, f[j] / base[j])
    for L, want in ((lam * 4.0 * (1 - 1e-9), 1.0), (lam * 1.0 * (1 + 1e-9), 1 / 16)):   # a hair outside: the same values
        sc = dict(rope_type="llama3", factor=16.0, low_freq_factor=1.0, high_freq_factor=4.0,
                  original_max_position_embeddings=L)
        for who, f in _both_frequency_tables(64, 500000.0, sc):
            assert abs(f[j] / base[j] - want) < 1e-7, (who, L, f[j] / base[j])


# ------------------------------------------------------------------ attention against a library routine
def _library_attention(q, k, v, scale, window=None):
    S, nh, hd = q.shape
    rep = nh // k.shape[1]
    kk, vv = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("shd,thd->hst", q, kk) * scale
    i = torch.arange(S)
    mask = i[None, :] > i[:, None]
    if window is not None:
        mask = mask | (i[None, :] < i[:, None] - window + 1)
    s = s.masked_fill(mask[None], float("-inf"))
    return torch.einsum("hst,thd->shd", torch.softmax(s, -1), vv)


@pytest.mark.parametrize("nh,nkv,window", [(4, 4, None), (4, 2, None), (6, 1, None), (4, 2, 5)])
def test_attention_reduces_to_softmax_qk_v(nh, nkv, window):
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(23, h, 16, generator=g) for h in (nh, nkv, nkv))
    got = P.attention(q, k, v, 0.25, window=window)
    assert torch.allclose(got, _library_attention(q, k, v, 0.25, window), atol=1e-5)


def test_attention_special_cases():
    g = torch.Generator().manual_seed(5)
    q, v = torch.randn(6, 2, 8, generator=g), torch.randn(6, 1, 8, generator=g)
    k = torch.randn(1, 1, 8, generator=g).expand(6, 1, 8)
    out = P.attention(q, k, v, 0.3)                      # equal keys: the running mean of the values
    for t in range(6):
        assert torch.allclose(out[t, 0], v[: t + 1, 0].mean(0), atol=1e-6)
    # consecutive query heads share a kv head (h // (heads / kv_heads)), not h % kv_heads
    q2, k2, v2 = torch.randn(4, 4, 8, generator=g), torch.randn(4, 2, 8, generator=g), torch.randn(4, 2, 8, generator=g)
    out2 = P.attention(q2, k2, v2, 0.3)
    solo = P.attention(q2[:, 1:2], k2[:, 0:1], v2[:, 0:1], 0.3)
    assert torch.allclose(out2[:, 1], solo[:, 0], atol=1e-6)


# ------------------------------------------------------------------ the whole model
def _tiny(raw, seed=0, std=0.1):
    from photon_infer_amd.config import LlamaConfig
    from photon_infer_amd.registry import build_model_spec
    from photon_infer_amd.weights import random_tensors
    cfg = LlamaConfig.from_dict(raw)
    return cfg.to_dict(), random_tensors(build_model_spec(cfg).tensor_specs(), seed, std, "uniform", torch.float32)


def test_model_is_causal_and_position_shift_invariant():
    cfg, W = _tiny(TINY_A)
    toks = torch.randint(0, 256, (12,), generator=torch.Generator().manual_seed(6)).tolist()
    full = P.llama_forward(cfg, W, toks)
    assert torch.allclose(P.llama_forward(cfg, W, toks[:7]), full[:7], atol=1e-5)   # later tokens are not seen
    # only distances count: shifting every position leaves the logits (up to float32 angles)
    shifted = P.llama_forward(cfg, W, toks, start_pos=17)
    assert torch.allclose(shifted, full, atol=2e-4)
    changed = P.llama_forward(cfg, W, toks[:3] + [(toks[3] + 1) % 256] + toks[4:])
    assert torch.allclose(changed[:3], full[:3], atol=1e-6) and not torch.allclose(changed[3:], full[3:], atol=1e-3)


def test_tied_and_untied_heads():
    cfg, W = _tiny(TINY_A)
    toks = [3, 1, 4, 1, 5]
    tied = P.llama_forward(cfg, W, toks)
    W2 = dict(W, **{"lm_head.weight": W["model.embed_tokens.weight"].clone()})
    assert torch.equal(P.llama_forward(dict(cfg, tie_word_embeddings=False), W2, toks), tied)
    W2["lm_head.weight"] = torch.zeros_like(W2["lm_head.weight"])
    assert P.llama_forward(dict(cfg, tie_word_embeddings=False), W2, toks).abs().max() == 0


def test_float64_agrees_with_float32():
    cfg, W = _tiny(TINY_B, seed=1, std=0.05)
    toks = torch.randint(0, 384, (40,), generator=torch.Generator().manual_seed(7)).tolist()
    a = P.llama_forward(cfg, W, toks)
    b = P.llama_forward(cfg, W, toks, dtype=torch.float64)
    assert (a.double() - b).abs().max() < 5e-5 * b.abs().max().clamp(min=1)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_whole_tensor_form_equals_the_loops(name):
    """``plain_wide`` (the same formulas over whole tensors, used where sequences are thousands of
    tokens long) against ``plain_llama``: with and without the bfloat16 rounding points, with a
    window, for all rows and for chosen rows, interleaved pairs too."""
    import plain_wide as PW
    from tiny_models import ALL

    raw, init = ALL[name]
    cfg, W = _tiny(raw, seed=3, std=init["std"])
    toks = torch.randint(0, raw["vocab_size"], (37,), generator=torch.Generator().manual_seed(8)).tolist()
    ref = P.llama_forward(cfg, W, toks)
    tol = 2e-5 * max(1.0, ref.abs().max().item())
    assert (PW.llama_forward(cfg, W, toks) - ref).abs().max() < tol
    assert (PW.llama_forward(cfg, W, toks, rows=[36, 0, 17]) - ref[[36, 0, 17]]).abs().max() < tol
    emu = P.llama_forward(cfg, W, toks, act_round=P.bf16_round)
    wide = PW.llama_forward(cfg, W, toks, act_round=P.bf16_round)
    # rounding points make the two forms differ where a value sits on a rounding boundary; the
    # deviation stays far below what the rounding itself does to the logits
    assert (wide - emu).abs().max() < 0.25 * (emu - ref).abs().max()
    win = P.llama_forward(cfg, W, toks, window=5)
    assert (PW.llama_forward(cfg, W, toks, window=5) - win).abs().max() < tol and (win - ref).abs().max() > 10 * tol
    inter = dict(cfg, rope_interleaved=True)
    assert (PW.llama_forward(inter, W, toks) - P.llama_forward(inter, W, toks)).abs().max() < tol
