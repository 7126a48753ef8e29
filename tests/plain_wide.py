"""The plain implementation's formulas over whole tensors instead of Python loops, for sequences
of a few thousand tokens at real layer sizes, where ``plain_llama`` would take minutes.

Test code only.  It has the same rounding points (``act_round``) and the same formulas, written
with library calls on whole tensors (a masked matrix of scores instead of a loop over tokens and
heads), on any device; ``tests/test_plain.py`` holds it to ``plain_llama`` on the tiny
configurations, which is what gives it its authority.  The output head is applied to the rows
asked for only.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional, Sequence

import torch

import plain_llama as P


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``plain_llama.rmsnorm`` for all rows at once."""
    rms = torch.sqrt((x * x).sum(-1, keepdim=True) / x.shape[1] + eps)
    return w * (x * (1.0 / rms))


def rope(x: torch.Tensor, positions: torch.Tensor, freqs, interleaved: bool) -> torch.Tensor:
    """``plain_llama.rope``: x [S, heads, head_dim], float32 angle from a float32 frequency."""
    half = len(freqs)
    f32 = torch.tensor(freqs, dtype=torch.float64).to(torch.float32).to(x.device)
    angle = (positions.to(torch.float32)[:, None] * f32[None, :]).to(x.dtype)       # [S, half]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    if interleaved:
        a, b = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
        out[..., 0:2 * half:2] = a * c - b * s
        out[..., 1:2 * half:2] = a * s + b * c
    else:
        a, b = x[..., :half], x[..., half:2 * half]
        out[..., :half] = a * c - b * s
        out[..., half:2 * half] = a * s + b * c
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int] = None,
              p_round: Optional[Callable] = None) -> torch.Tensor:
    """``plain_llama.attention``: q [S, heads, hd], k / v [S, kv_heads, hd]; token t sees keys
    max(0, t - W + 1) .. t of kv head h // (heads / kv_heads)."""
    S, nh, hd = q.shape
    kv_mul = nh // k.shape[1]
    kk = k.repeat_interleave(kv_mul, dim=1)                    # head h reads kv head h // kv_mul
    vv = v.repeat_interleave(kv_mul, dim=1)
    scores = torch.einsum("shd,thd->hst", q, kk) * scale       # [heads, query, key]
    t = torch.arange(S, device=q.device)
    hidden = t[None, :] > t[:, None]
    if window is not None:
        hidden = hidden | (t[None, :] < t[:, None] - window + 1)
    scores = scores.masked_fill(hidden[None], float("-inf"))
    e = torch.exp(scores - scores.amax(-1, keepdim=True))
    weights = p_round(e) if p_round is not None else e
    out = torch.einsum("hst,thd->shd", weights, vv) / e.sum(-1).transpose(0, 1)[..., None]
    return out


def llama_forward(config: dict, tensors: Dict[str, torch.Tensor], token_ids: Sequence[int], rows: Optional[Sequence[int]] = None,
                  act_round: Optional[Callable] = None, device="cpu", window: Optional[int] = None) -> torch.Tensor:
    """Float32 logits [len(rows), vocab] (all rows when ``rows`` is None) of one whole sequence;
    the order of ``plain_llama.llama_forward``."""
    rd = act_round or (lambda t: t)
    dev = torch.device(device)

    def W(name):
        return tensors[name].to(device=dev, dtype=torch.float32)

    D = config["hidden_size"]
    nh = config["num_attention_heads"]
    nkv = config.get("num_key_value_heads") or nh
    hd = config.get("head_dim") or D // nh
    eps = config["rms_norm_eps"]
    freqs = P.rope_frequencies(hd, config.get("rope_theta", 10000.0), config.get("rope_scaling"))
    interleaved = bool(config.get("rope_interleaved", False))
    S = len(token_ids)
    positions = torch.arange(S, device=dev)
    scale = 1.0 / math.sqrt(hd)
    x = W("model.embed_tokens.weight")[torch.tensor(list(token_ids), device=dev)]
    for i in range(config["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rd(rmsnorm(x, W(p + "input_layernorm.weight"), eps))
        q = rd(h @ W(p + "self_attn.q_proj.weight").t()).reshape(S, nh, hd)
        k = rd(h @ W(p + "self_attn.k_proj.weight").t()).reshape(S, nkv, hd)
        v = rd(h @ W(p + "self_attn.v_proj.weight").t()).reshape(S, nkv, hd)
        q = rd(rope(q, positions, freqs, interleaved))
        k = rd(rope(k, positions, freqs, interleaved))
        a = rd(attention(q, k, v, scale, window, act_round).reshape(S, nh * hd))
        x = x + a @ W(p + "self_attn.o_proj.weight").t()
        h = rd(rmsnorm(x, W(p + "post_attention_layernorm.weight"), eps))
        g = rd(h @ W(p + "mlp.gate_proj.weight").t())
        u = rd(h @ W(p + "mlp.up_proj.weight").t())
        x = x + rd(P.swiglu(g, u)) @ W(p + "mlp.down_proj.weight").t()
    if rows is not None:
        x = x[torch.tensor(list(rows), device=dev)]
    h = rd(rmsnorm(x, W("model.norm.weight"), eps))
    head = W("model.embed_tokens.weight" if config.get("tie_word_embeddings", False) else "lm_head.weight")
    return h @ head.t()
