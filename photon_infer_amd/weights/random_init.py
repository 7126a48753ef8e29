"""Random-weights mode: write a model folder from a configuration and a seed.

The reference has this only as a test helper (tests/model/test_llama_model.cpp:31-42:
``mt19937(seed)``, N(0, 0.02) for every tensor).  Here each tensor has its own stream,
keyed by (seed, tensor name), so a tensor's values do not depend on which other
tensors exist or in which order they are made.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterable

import torch

from ..registry import build_model_spec
from .loader import TensorSpec
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_tensors(specs: Iterable[TensorSpec], seed: int, std: float = 0.02, norm_init: str = "ones",
                   dtype: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """``norm_init``: "ones" or "uniform" (U(0.5, 1.5))."""
    out = {}
    for s in specs:
        g = _generator(seed, s.name)
        if s.role == "norm":
            t = torch.ones(s.shape) if norm_init == "ones" else torch.rand(s.shape, generator=g) + 0.5
        elif s.role == "int_table":
            out[s.name] = torch.randint(0, 2**15, s.shape, generator=g, dtype=torch.int32)
            continue
        else:
            t = torch.randn(s.shape, generator=g, dtype=torch.float32) * std
        out[s.name] = t.to(dtype)
    return out


def write_random_model(config, out_dir: str, seed: int = 0, std: float = 0.02, norm_init: str = "ones",
                       dtype: str | None = None) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` into ``out_dir``."""
    name = dtype or getattr(config, "torch_dtype", "bfloat16")
    if name not in _DTYPES:
        raise ValueError(f"storage dtype '{name}' is not one of {sorted(_DTYPES)}")
    os.makedirs(out_dir, exist_ok=True)
    spec = build_model_spec(config)
    tensors = random_tensors(spec.tensor_specs(), seed, std, norm_init, _DTYPES[name])
    raw = config.to_dict()
    raw["torch_dtype"] = name
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=2)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      {"format": "pt", "seed": str(seed), "std": str(std), "norm_init": norm_init})
    return out_dir


def random_model_folder(config_path: str, seed: int = 0, std: float = 0.02, norm_init: str = "ones") -> str:
    """A fresh temporary model folder with random weights for the bare configuration at
    ``config_path`` (a config.json file, or a folder that holds one).  The caller removes it."""
    import tempfile

    from ..registry import config_from_dict

    path = os.path.join(config_path, "config.json") if os.path.isdir(config_path) else config_path
    with open(path, encoding="utf-8") as f:
        config = config_from_dict(json.load(f), path)
    return write_random_model(config, tempfile.mkdtemp(prefix="photon_random_"), seed=seed, std=std, norm_init=norm_init)
