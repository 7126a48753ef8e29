"""Llama: the layer list that its configuration describes.

Block order and tensor roles follow src/arch/transformer_block.cpp:189-299 and
src/arch/llama_model.cpp:186-272: embedding, N x [RMSNorm, GQA attention with rotary
positions, residual, RMSNorm, SwiGLU, residual], final RMSNorm, output head (tied to
the embedding or its own).  Tensor names are those of a Llama model folder; the
reference's operator names map as wq/wk/wv/wo -> self_attn.{q,k,v,o}_proj,
w1/w3/w2 -> mlp.{gate,up,down}_proj, attn_norm/ffn_norm ->
input_layernorm/post_attention_layernorm (src/io/checkpoint.cpp:256-289).
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS
from ..parts.embedding import LMHead, TokenEmbedding
from ..parts.model import ModelSpec
from ..registry import register_architecture


def build_llama(cfg: LlamaConfig) -> ModelSpec:
    rope = POSITION_ENCODINGS.make(
        "rope", head_dim=cfg.head_dim, theta=cfg.rope_theta, scaling=cfg.rope_scaling,
        interleaved=cfg.rope_interleaved,
    )
    layers = []
    for i in range(cfg.num_hidden_layers):
        block = BLOCKS.make(
            "prenorm",
            norm1=("input_layernorm.", NORMS.make("rmsnorm", dim=cfg.hidden_size, eps=cfg.rms_norm_eps)),
            mixer=("self_attn.", MIXERS.make(
                "attention", hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
                num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim, position=rope)),
            norm2=("post_attention_layernorm.", NORMS.make("rmsnorm", dim=cfg.hidden_size, eps=cfg.rms_norm_eps)),
            ffn=("mlp.", FEED_FORWARDS.make(
                "swiglu", hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                activation=cfg.hidden_act)),
        )
        layers.append((f"model.layers.{i}.", block))
    ignorable = ["*.rotary_emb.inv_freq"]
    if cfg.tie_word_embeddings:
        ignorable.append("lm_head.weight")
    return ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=("model.embed_tokens.", TokenEmbedding(cfg.vocab_size, cfg.hidden_size)),
        layers=layers,
        final_norm=("model.norm.", NORMS.make("rmsnorm", dim=cfg.hidden_size, eps=cfg.rms_norm_eps)),
        head=("lm_head.", LMHead(cfg.vocab_size, cfg.hidden_size, tied=cfg.tie_word_embeddings)),
        ignorable=tuple(ignorable),
        eos_token_ids=tuple(cfg.eos_token_ids),
        bos_token_id=cfg.bos_token_id,
    )


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama)
