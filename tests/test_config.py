"""Configuration and registry (CPU)."""
import json
import os

import pytest

from photon_infer_amd import (ConfigError, UnsupportedModelError, build_model_spec, get_architecture, load_config,
                              register_architecture, registered_architectures)
from photon_infer_amd.config import LlamaConfig
from tiny_models import TINY_A, TINY_B, TINY_C


def test_llama_config_reads_every_key():
    cfg = LlamaConfig.from_dict(TINY_B)
    assert (cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (128, 320, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (4, 1, 32)
    assert cfg.vocab_size == 384 and cfg.max_position_embeddings == 256
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 500000.0
    assert cfg.rope_scaling.rope_type == "llama3" and cfg.rope_scaling.factor == 8.0
    assert cfg.rope_scaling.original_max_position_embeddings == 64
    assert cfg.tie_word_embeddings is False
    assert cfg.q_size == 128 and cfg.kv_size == 32 and cfg.queries_per_kv == 4


def test_defaults_follow_the_reference():
    # head_size = dim / head_num (src/arch/config.cpp:27), kv heads default to heads
    raw = dict(TINY_A)
    raw.pop("num_key_value_heads")
    cfg = LlamaConfig.from_dict(raw)
    assert cfg.head_dim == 16 and cfg.num_key_value_heads == 4
    assert cfg.rope_scaling is None and cfg.rope_theta == 10000.0


def test_head_dim_need_not_divide_hidden():
    cfg = LlamaConfig.from_dict(TINY_C)
    assert cfg.head_dim * cfg.num_attention_heads != cfg.hidden_size
    assert cfg.rope_scaling.rope_type == "linear"


def test_round_trip_through_config_json(tmp_path):
    for raw in (TINY_A, TINY_B, TINY_C):
        cfg = LlamaConfig.from_dict(raw)
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        assert load_config(str(tmp_path)) == cfg


def test_eos_may_be_a_list():
    cfg = LlamaConfig.from_dict(dict(TINY_A, eos_token_id=[5, 7], bos_token_id=1))
    assert cfg.eos_token_ids == (5, 7) and cfg.bos_token_id == 1
    assert LlamaConfig.from_dict(dict(TINY_A, eos_token_id=9)).eos_token_ids == (9,)


@pytest.mark.parametrize("change, err", [
    (dict(hidden_size=None), ConfigError),
    (dict(num_attention_heads=0), ConfigError),
    (dict(num_attention_heads=4, num_key_value_heads=3), ConfigError),
    (dict(hidden_size=66), ConfigError),                      # not divisible by heads, no head_dim
    (dict(head_dim=15), ConfigError),
    (dict(rms_norm_eps="small"), ConfigError),
    (dict(vocab_size=-1), ConfigError),
    (dict(hidden_act="gelu"), UnsupportedModelError),
    (dict(attention_bias=True), UnsupportedModelError),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 2.0}), UnsupportedModelError),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 2.0}), ConfigError),   # constants missing
    (dict(architectures=[]), ConfigError),
])
def test_rejected_values(change, err):
    raw = dict(TINY_A)
    raw.update(change)
    with pytest.raises(err):
        LlamaConfig.from_dict(raw)


def test_errors_name_the_key():
    raw = dict(TINY_A)
    del raw["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        LlamaConfig.from_dict(raw)


def test_registry_lookup_and_unknown_architecture(tmp_path):
    assert "LlamaForCausalLM" in registered_architectures()
    assert get_architecture("LlamaForCausalLM").config_cls is LlamaConfig
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, architectures=["MambaForCausalLM"])))
    with pytest.raises(UnsupportedModelError, match="MambaForCausalLM"):
        load_config(str(tmp_path))


def test_missing_and_malformed_config_json(tmp_path):
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))


def test_model_spec_is_data():
    spec = build_model_spec(LlamaConfig.from_dict(TINY_B))
    assert len(spec.layers) == 3 and [e.layer for e in spec.run_order] == [0, 1, 2]
    names = {s.name: s.shape for s in spec.tensor_specs()}
    assert names["model.layers.2.self_attn.k_proj.weight"] == (32, 128)
    assert names["model.layers.0.mlp.down_proj.weight"] == (128, 320)
    assert names["lm_head.weight"] == (384, 128)
    tied = build_model_spec(LlamaConfig.from_dict(TINY_A))
    assert "lm_head.weight" not in {s.name for s in tied.tensor_specs()}


def test_another_architecture_can_be_registered():
    class ToyConfig:
        architecture = "ToyForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls()

    register_architecture("ToyForCausalLM", ToyConfig, lambda cfg: "spec")
    assert build_model_spec(ToyConfig()) == "spec"
