"""Tiny Llama configurations for tests; they differ in every size and option."""
from __future__ import annotations

import os

import torch

from photon_infer_amd.config import LlamaConfig
from photon_infer_amd.weights import write_random_model

TINY_A = dict(
    architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=176, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, vocab_size=256, max_position_embeddings=128,
    rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True,
)
TINY_A_INIT = dict(std=0.02, norm_init="ones", block_size=4)

TINY_B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=128, intermediate_size=320, num_hidden_layers=3,
    num_attention_heads=4, num_key_value_heads=1, head_dim=32, vocab_size=384, max_position_embeddings=256,
    rms_norm_eps=1e-6, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    tie_word_embeddings=False,
)
TINY_B_INIT = dict(std=0.05, norm_init="uniform", block_size=8)

# head_dim * heads != hidden, 3 heads in 3 groups, widths that are no power of two, a
# vocabulary that is no multiple of anything, linear frequency scaling, bigger weights so
# attention is far from uniform
TINY_C = dict(
    architectures=["LlamaForCausalLM"], hidden_size=96, intermediate_size=200, num_hidden_layers=4,
    num_attention_heads=6, num_key_value_heads=3, head_dim=48, vocab_size=1001, max_position_embeddings=512,
    rms_norm_eps=3e-5, rope_theta=1000.0, rope_scaling=dict(rope_type="linear", factor=2.0),
    tie_word_embeddings=False,
)
TINY_C_INIT = dict(std=0.12, norm_init="uniform", block_size=16)

# sizes the matrix-core kernels take (head_dim 64, pages of 16, widths in multiples of 8), so
# that the bfloat16 engine runs them: 2 heads per kv head, llama3 scaling with a short context
TINY_D = dict(
    architectures=["LlamaForCausalLM"], hidden_size=128, intermediate_size=272, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, head_dim=64, vocab_size=520, max_position_embeddings=2048,
    rms_norm_eps=1e-5, rope_theta=50000.0,
    rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=128),
    tie_word_embeddings=True,
)
TINY_D_INIT = dict(std=0.08, norm_init="uniform", block_size=16)

# the other head size of the matrix-core kernels (128), four heads on one kv head, pages of 32,
# an untied head, no scaling of the rotation
TINY_E = dict(
    architectures=["LlamaForCausalLM"], hidden_size=160, intermediate_size=344, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=1, head_dim=128, vocab_size=776, max_position_embeddings=512,
    rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=False,
)
TINY_E_INIT = dict(std=0.06, norm_init="uniform", block_size=32)

# Large enough that the kernels chosen at real sizes run inside the model: products whose k-range
# is split (o, down and q|k|v: hidden >= 1024 and intermediate >= 2816 give K // 256 >= 2 and
# K // 512 >= 2), their pieces added by the next norm, by the rotation and by the fused decode
# kernel; four heads per kv head at head size 64; a vocabulary the two-kernel sampler takes; the
# frequency scaling constants of the 1B model
TINY_F = dict(
    architectures=["LlamaForCausalLM"], hidden_size=1024, intermediate_size=2816, num_hidden_layers=2,
    num_attention_heads=16, num_key_value_heads=4, head_dim=64, vocab_size=32768, max_position_embeddings=1024,
    rms_norm_eps=1e-5, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True,
)
TINY_F_INIT = dict(std=0.03, norm_init="uniform", block_size=16)

# a head size of 96: three fragments of 32 features in the matrix-core attention kernels (tile
# kernel and key-split decode kernel; the decode kernel that starts from the projection takes
# 64 and 128 only, so single tokens go through the separate rotation kernel)
TINY_G = dict(
    architectures=["LlamaForCausalLM"], hidden_size=160, intermediate_size=264, num_hidden_layers=2,
    num_attention_heads=3, num_key_value_heads=1, head_dim=96, vocab_size=600, max_position_embeddings=512,
    rms_norm_eps=1e-5, rope_theta=20000.0, tie_word_embeddings=True,
)
TINY_G_INIT = dict(std=0.07, norm_init="uniform", block_size=16)

# H: a head of 160 features, above what two rounds of 128 keys allow in the LDS: prompts go
# through the tile kernel in rounds of 64 keys with 16 columns per wave; two heads on one kv head
TINY_H = dict(
    architectures=["LlamaForCausalLM"], hidden_size=112, intermediate_size=200, num_hidden_layers=2,
    num_attention_heads=2, num_key_value_heads=1, head_dim=160, vocab_size=410, max_position_embeddings=512,
    rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=False,
)
TINY_H_INIT = dict(std=0.06, norm_init="uniform", block_size=16)

ALL = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT), "D": (TINY_D, TINY_D_INIT),
       "E": (TINY_E, TINY_E_INIT), "F": (TINY_F, TINY_F_INIT),
       "G": (TINY_G, TINY_G_INIT), "H": (TINY_H, TINY_H_INIT)}


def make_model_dir(tmp_path, name: str, seed: int = 0, storage: str = "bfloat16") -> str:
    raw, init = ALL[name]
    cfg = LlamaConfig.from_dict(raw)
    d = os.path.join(str(tmp_path), f"tiny_{name}_{seed}_{storage}")
    write_random_model(cfg, d, seed=seed, std=init["std"], norm_init=init["norm_init"], dtype=storage)
    return d


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
