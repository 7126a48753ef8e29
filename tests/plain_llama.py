"""A plain, slow implementation of the Llama forward pass: whole sequences, no cache.

Written from the reference's formulas (each function cites file:line in the reference
repository, lumia431/photon_infer); it shares no code with ``photon_infer_amd``.  Everything is explicit
torch arithmetic on the CPU in float32 (or float64 when asked), one function per part.

``act_round`` lets a test emulate the places where the bfloat16 path rounds
activations (after a norm, after a projection, after the rotation, the attention
probabilities for the value product, the attention output, the gated product), so the
bfloat16 engine can be compared tightly instead of with a loose bound.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Callable, Dict, List, Optional

import torch


# ---------------------------------------------------------------------------------- files
_ST = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "I32": torch.int32, "I64": torch.int64}


def read_model_folder(model_dir: str):
    """(config dict, {name: float tensor}) of a folder with config.json + model.safetensors."""
    with open(os.path.join(model_dir, "config.json")) as f:
        config = json.load(f)
    tensors = {}
    with open(os.path.join(model_dir, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        payload = f.read()
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        t = torch.frombuffer(bytearray(payload[b:e]), dtype=_ST[info["dtype"]]).reshape(info["shape"])
        tensors[name] = t
    return config, tensors


# ---------------------------------------------------------------------------------- parts
def embedding(table: torch.Tensor, ids) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] (src/ops/kernels/cuda/embedding_kernel.cu:31-63)."""
    return torch.stack([table[int(i)] for i in ids])


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """include/photon/ops/kernels/rmsnorm_kernel.hpp:55-87: mean of squares over the row,
    rms = sqrt(mean + eps), out = w * (x / rms)."""
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        mean_sq = (x[t] * x[t]).sum() / x.shape[1]
        rms = torch.sqrt(mean_sq + eps)
        out[t] = w * (x[t] * (1.0 / rms))
    return out


def linear(x: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
    """include/photon/ops/kernels/matmul_kernel.hpp:94-129: out[b, i] = sum_j x[b, j] * W[i, j]
    (weights [out, in], no bias)."""
    return x @ W.t()


def rope_frequencies(rotary_dim: int, theta: float, scaling: Optional[dict]) -> List[float]:
    """Per-pair frequencies in double precision.

    Base: include/photon/ops/kernels/rope_kernel.hpp:67-83, freq = 1 / theta^(d / head_size)
    for the even index d = 2j (the reference has theta = 10000).  The llama3 rule is not in
    the reference; it is the piecewise rule stated in the model family's config keys:
    wavelength lam = 2 pi / f; lam < L/high keeps f; lam > L/low gives f/factor; otherwise
    s = (L/lam - low) / (high - low), f = (1 - s) f/factor + s f.
    """
    freqs = []
    for j in range(rotary_dim // 2):
        f = 1.0 / (theta ** ((2 * j) / rotary_dim))
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type"))
            if kind == "llama3":
                factor = scaling["factor"]
                low, high = scaling["low_freq_factor"], scaling["high_freq_factor"]
                L = scaling["original_max_position_embeddings"]
                lam = 2.0 * math.pi / f
                if lam < L / high:
                    pass
                elif lam > L / low:
                    f = f / factor
                else:
                    s = (L / lam - low) / (high - low)
                    f = (1.0 - s) * f / factor + s * f
            elif kind == "linear":
                f = f / scaling["factor"]
            elif kind not in (None, "default"):
                raise ValueError(kind)
        freqs.append(f)
    return freqs


def rope(x: torch.Tensor, positions, freqs: List[float], interleaved: bool) -> torch.Tensor:
    """include/photon/ops/kernels/rope_kernel.hpp:126-165: each pair (a, b) of a head becomes
    (a cos - b sin, a sin + b cos) with angle = pos * f_j.  ``interleaved`` pairs
    (x[2j], x[2j+1]) as the reference does; otherwise (x[j], x[j + R/2]), the layout of
    Llama model folders.  The angle is formed in float32 from a float32 frequency.
    x: [S, heads, head_dim]; dims beyond the rotated width pass through."""
    out = x.clone()
    half = len(freqs)
    f32 = torch.tensor(freqs, dtype=torch.float64).to(torch.float32)
    for t in range(x.shape[0]):
        angle = (torch.tensor(float(positions[t]), dtype=torch.float32) * f32).to(x.dtype)
        c, s = torch.cos(angle), torch.sin(angle)
        for j in range(half):
            i0, i1 = (2 * j, 2 * j + 1) if interleaved else (j, j + half)
            a, b = x[t, :, i0], x[t, :, i1]
            out[t, :, i0] = a * c[j] - b * s[j]
            out[t, :, i1] = a * s[j] + b * c[j]
    return out


def softmax(scores: torch.Tensor) -> torch.Tensor:
    """include/photon/ops/kernels/mha_kernel.hpp:36-55: subtract the max, exponentiate,
    divide by the sum (nothing added to the denominator)."""
    e = torch.exp(scores - scores.max())
    return e / e.sum()


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, positions=None,
              window: Optional[int] = None, p_round: Optional[Callable] = None) -> torch.Tensor:
    """include/photon/ops/kernels/mha_kernel.hpp:174-230: for the query at position p and head
    h, kv head = h // (heads / kv_heads); score_t = <q, k_t> * scale for t = 0..p; softmax;
    out = sum_t P_t v_t.  ``window`` W restricts t to p-W+1..p.
    q: [S, heads, hd], k/v: [S, kv_heads, hd] -> [S, heads, hd]."""
    S, nh, hd = q.shape
    kv_mul = nh // k.shape[1]
    out = torch.zeros_like(q)
    for t in range(S):
        lo = 0 if window is None else max(0, t - window + 1)
        for h in range(nh):
            g = h // kv_mul
            scores = (k[lo:t + 1, g, :] * q[t, h, :]).sum(-1) * scale
            p = softmax(scores)
            if p_round is not None:
                # the matrix-core kernel rounds unnormalised probabilities; the effect is
                # the same relative rounding of each weight
                e = torch.exp(scores - scores.max())
                out[t, h, :] = (p_round(e).unsqueeze(-1) * v[lo:t + 1, g, :]).sum(0) / e.sum()
            else:
                out[t, h, :] = (p.unsqueeze(-1) * v[lo:t + 1, g, :]).sum(0)
    return out


def swiglu(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """include/photon/ops/kernels/swiglu_kernel.hpp:52-76: silu(g) * u, silu(x) = x / (1 + exp(-x))."""
    return g / (1.0 + torch.exp(-g)) * u


def argmax(logits: torch.Tensor) -> int:
    """src/arch/llama_model.cpp:304-328: strict '>' scan, the first maximum wins."""
    best, idx = logits[0], 0
    for i in range(1, logits.shape[0]):
        if logits[i] > best:
            best, idx = logits[i], i
    return idx


def sample_temperature(logits: torch.Tensor, temperature: float, u: float) -> int:
    """demo/llama_infer.cpp:77-101: p = exp((l - max) / T) / sum; first i with u <= cumsum."""
    p = torch.exp((logits - logits.max()) / temperature)
    p = p / p.sum()
    cum = 0.0
    for i in range(p.shape[0]):
        cum += float(p[i])
        if u <= cum:
            return i
    nz = torch.nonzero(p > 0)
    return int(nz[-1])


# ---------------------------------------------------------------------------------- the model
def llama_forward(config: dict, tensors: Dict[str, torch.Tensor], token_ids, dtype=torch.float32,
                  act_round: Optional[Callable] = None, start_pos: int = 0,
                  window: Optional[int] = None) -> torch.Tensor:
    """Logits [S, vocab] of one whole sequence.

    Order per layer (src/arch/transformer_block.cpp:189-299): norm -> q,k,v -> rotation ->
    attention -> o projection -> residual add -> norm -> gate, up -> SwiGLU -> down ->
    residual add; then the final norm and the output head (src/arch/llama_model.cpp:242-256).
    """
    rd = act_round or (lambda t: t)
    W = {n: t.to(dtype) for n, t in tensors.items()}
    D = config["hidden_size"]
    nh = config["num_attention_heads"]
    nkv = config.get("num_key_value_heads") or nh
    hd = config.get("head_dim") or D // nh
    eps = config["rms_norm_eps"]
    freqs = rope_frequencies(hd, config.get("rope_theta", 10000.0), config.get("rope_scaling"))
    interleaved = bool(config.get("rope_interleaved", False))
    S = len(token_ids)
    positions = list(range(start_pos, start_pos + S))
    scale = 1.0 / math.sqrt(hd)

    x = embedding(W["model.embed_tokens.weight"], token_ids)
    for i in range(config["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rd(rmsnorm(x, W[p + "input_layernorm.weight"], eps))
        q = rd(linear(h, W[p + "self_attn.q_proj.weight"])).reshape(S, nh, hd)
        k = rd(linear(h, W[p + "self_attn.k_proj.weight"])).reshape(S, nkv, hd)
        v = rd(linear(h, W[p + "self_attn.v_proj.weight"])).reshape(S, nkv, hd)
        q = rd(rope(q, positions, freqs, interleaved))
        k = rd(rope(k, positions, freqs, interleaved))
        a = rd(attention(q, k, v, scale, window=window, p_round=act_round).reshape(S, nh * hd))
        x = x + linear(a, W[p + "self_attn.o_proj.weight"])
        h = rd(rmsnorm(x, W[p + "post_attention_layernorm.weight"], eps))
        g = rd(linear(h, W[p + "mlp.gate_proj.weight"]))
        u = rd(linear(h, W[p + "mlp.up_proj.weight"]))
        x = x + linear(rd(swiglu(g, u)), W[p + "mlp.down_proj.weight"])
    h = rd(rmsnorm(x, W["model.norm.weight"], eps))
    head = W["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else W["lm_head.weight"]
    return linear(h, head)


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def greedy_generate(config: dict, tensors, prompt: List[int], n_new: int, dtype=torch.float32) -> List[int]:
    """Feed the whole sequence again for every new token (no cache) and take the argmax."""
    seq = list(prompt)
    out = []
    for _ in range(n_new):
        logits = llama_forward(config, tensors, seq, dtype)
        nxt = argmax(logits[-1])
        out.append(nxt)
        seq.append(nxt)
    return out
