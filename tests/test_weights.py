"""Safetensors reading, the single listing error, storage dtypes, random-weights mode (CPU)."""
import json
import os
import struct

import pytest
import torch

from photon_infer_amd import WeightError, build_model_spec, load_config
from photon_infer_amd.config import LlamaConfig
from photon_infer_amd.errors import FileFormatError
from photon_infer_amd.weights import (SafetensorsFile, load_model_tensors, storage_dtype, write_random_model,
                                      write_safetensors)
from tiny_models import TINY_A, TINY_B, make_model_dir


def test_safetensors_round_trip(tmp_path):
    tensors = {
        "a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int64).reshape(2, 3),
        "empty": torch.zeros(0, 4),
    }
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, {"k": "v"})
    with SafetensorsFile(path) as f:
        assert set(f.names()) == set(tensors) and f.metadata == {"k": "v"}
        for n, t in tensors.items():
            got = f.read(n)
            assert got.dtype == t.dtype and got.shape == t.shape and torch.equal(got, t)


def test_third_party_reader_agrees(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    d = make_model_dir(tmp_path, "A", seed=1)
    theirs = st.load_file(os.path.join(d, "model.safetensors"))
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        assert set(theirs) == set(f.names())
        for n in theirs:
            assert torch.equal(theirs[n], f.read(n))


def test_truncated_and_malformed_files(tmp_path):
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, {"a": torch.randn(64, 64)})
    blob = open(path, "rb").read()
    open(path, "wb").write(blob[:-100])
    with pytest.raises(FileFormatError, match="truncated"):
        SafetensorsFile(path)
    open(path, "wb").write(struct.pack("<Q", 10**12) + b"{}")
    with pytest.raises(FileFormatError, match="header length"):
        SafetensorsFile(path)
    open(path, "wb").write(b"abc")
    with pytest.raises(FileFormatError):
        SafetensorsFile(path)
    with pytest.raises(FileFormatError):
        SafetensorsFile(str(tmp_path / "missing.safetensors"))


def test_storage_dtype_policy():
    bf, f32 = torch.bfloat16, torch.float32
    assert storage_dtype(torch.bfloat16, bf) == bf
    assert storage_dtype(torch.float16, bf) == bf
    assert storage_dtype(torch.float32, bf) == f32          # stored in 32-bit stays so
    assert storage_dtype(torch.bfloat16, f32) == f32        # the float32 mode widens everything
    assert storage_dtype(torch.int64, bf) == torch.int32    # integer tables as int32


def _specs(raw):
    return build_model_spec(LlamaConfig.from_dict(raw))


def test_loads_by_name_and_keeps_dtypes(tmp_path):
    d = make_model_dir(tmp_path, "B", seed=2)
    spec = build_model_spec(load_config(d))
    got = load_model_tensors(d, spec.tensor_specs(), torch.bfloat16, "cpu", spec.ignorable)
    assert set(got) == {s.name for s in spec.tensor_specs()}
    assert all(t.dtype == torch.bfloat16 for t in got.values())
    got32 = load_model_tensors(d, spec.tensor_specs(), torch.float32, "cpu", spec.ignorable)
    assert all(t.dtype == torch.float32 for t in got32.values())
    for n in got:
        assert torch.equal(got[n].float(), got32[n])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=3)
    path = os.path.join(d, "model.safetensors")
    with SafetensorsFile(path) as f:
        tensors = {n: f.read(n) for n in f.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 32, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rogue.weight"] = torch.zeros(2, 2)
    write_safetensors(path, tensors)
    spec = _specs(TINY_A)
    with pytest.raises(WeightError) as ei:
        load_model_tensors(d, spec.tensor_specs(), torch.bfloat16, "cpu", spec.ignorable)
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rogue.weight"]
    assert e.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (64, 64), (64, 32))]
    text = str(e)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (1)", "rogue", "up_proj", "[64, 32]"):
        assert needle in text


def test_tied_head_ignores_a_stored_lm_head_but_untied_needs_it(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=4)
    path = os.path.join(d, "model.safetensors")
    with SafetensorsFile(path) as f:
        tensors = {n: f.read(n) for n in f.names()}
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(path, tensors)
    spec = _specs(TINY_A)
    got = load_model_tensors(d, spec.tensor_specs(), torch.bfloat16, "cpu", spec.ignorable)
    assert "lm_head.weight" not in got
    untied = _specs(dict(TINY_A, tie_word_embeddings=False))
    del tensors["lm_head.weight"]
    write_safetensors(path, tensors)
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_model_tensors(d, untied.tensor_specs(), torch.bfloat16, "cpu", untied.ignorable)


def test_missing_weight_file(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    spec = _specs(TINY_A)
    with pytest.raises(FileFormatError, match="model.safetensors"):
        load_model_tensors(str(tmp_path), spec.tensor_specs(), torch.bfloat16, "cpu")


def test_random_mode_is_seeded_per_tensor(tmp_path):
    a = make_model_dir(tmp_path / "1", "B", seed=7)
    b = make_model_dir(tmp_path / "2", "B", seed=7)
    c = make_model_dir(tmp_path / "3", "B", seed=8)
    fa, fb, fc = (SafetensorsFile(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    n = "model.layers.1.mlp.gate_proj.weight"
    assert torch.equal(fa.read(n), fb.read(n)) and not torch.equal(fa.read(n), fc.read(n))
    # a tensor's values do not depend on which other tensors exist: 2 layers vs 3 layers
    cfg2 = LlamaConfig.from_dict(dict(TINY_B, num_hidden_layers=2))
    d2 = write_random_model(cfg2, str(tmp_path / "4"), seed=7, std=0.05, norm_init="uniform")
    with SafetensorsFile(os.path.join(d2, "model.safetensors")) as f2:
        assert torch.equal(f2.read(n), fa.read(n))
    w = fa.read(n).float()
    assert abs(w.std().item() - 0.05) < 0.005 and abs(w.mean().item()) < 0.005
    nw = fa.read("model.norm.weight").float()
    assert 0.5 <= nw.min().item() and nw.max().item() <= 1.5 and nw.std().item() > 0.1
    with SafetensorsFile(os.path.join(make_model_dir(tmp_path / "5", "A"), "model.safetensors")) as f5:
        assert torch.equal(f5.read("model.norm.weight").float(), torch.ones(64))
    for f in (fa, fb, fc):
        f.close()


def test_random_mode_can_store_float32(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=1, storage="float32")
    assert load_config(d).torch_dtype == "float32"
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        assert f.read("model.embed_tokens.weight").dtype == torch.float32
