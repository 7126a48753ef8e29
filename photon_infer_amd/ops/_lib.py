"""ctypes binding of the kernel libraries.  Loading fails loudly; nothing falls back."""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p
from typing import Dict

import torch

from ..errors import KernelError, KernelLibraryMissing
from . import build

P, I, L, F = c_void_p, c_int, c_long, c_float

# entry point -> argument types (all return int: 0 = ok)
_SIGNATURES = {
    "core": {
        "pi_embedding": [P, P, I, P, I, I, I, P],
        "pi_rmsnorm": [P, I, P, P, P, I, F, I, I, P, I, L, P],
        "pi_swiglu": [P, P, I, I, I, I, P],
        "pi_rope_kv_write": [P, L, P, L, P, L, I, P, P, P, I, I, I, I, I, I, I, P, P, P, I, I, L, P, I, I, I, I, I, P],
        "pi_gemm_general": [P, I, L, P, I, L, P, I, L, I, I, I, I, P],
        "pi_paged_attention_general": [P, L, P, L, P, P, I, P, I, P, P, I, I, I, I, I, F, I, L, I, P, L, P],
        "pi_paged_attention_general_ranges": [I, I, I],
        "pi_rope_table": [P, P, P, I, I, P],
        "pi_sample": [P, P, L, P, P, I, I, P, L, P],
        "pi_sample_static": [P, P, L, P, P, I, I, P],
    },
    "bf16": {
        "pi_gemm_mfma": [P, I, L, P, L, P, L, I, I, I, I, P],
        "pi_gemm_mfma_pieces": [I, I],
        "pi_gemm_skinny": [P, I, L, P, L, P, L, I, I, I, I, P, L, P, I, P],
        "pi_splitk_reduce": [P, I, L, P, I, I, I, P],
        "pi_attention_tile_rows": [I, I, I],
        "pi_attention_prefill_mfma": [P, L, P, L, P, P, P, I, P, P, P, P, P, P, P, P, I, I, I, I, I, I, F, I, L, P],
        "pi_attention_combine_rows": [P, L, P, I, P, I, I, I, P],
        "pi_attention_decode": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, F, I, L, I, P, L, P],
        "pi_attention_decode_fused": [P, L, P, L, P, I, I, I, P, I, P, P, P, I, P, P, I, I, I, I, I, F, I, L, I, P, L, I, P],
        "pi_gemm_skinny_ranges": [P, I, L, P, I, I, I, P, L, I, I, I, P, L, P, I, P],
    },
}

_LIBS: Dict[str, ctypes.CDLL] = {}


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_CURRENT_DEVICE = getattr(torch._C, "_cuda_getDevice", None)


def current_stream() -> int:
    """The handle of torch's current HIP stream on the current device (whoever launches kernels
    for tensors of another device makes that device current first; ``ModelRunner`` does).  Asked
    for at every kernel launch (a step of a few hundred launches), so by the shortest way torch
    offers: its Python-level ``current_stream()`` costs as much as the launch itself."""
    if _RAW_STREAM is None or _CURRENT_DEVICE is None:
        return torch.cuda.current_stream().cuda_stream
    return _RAW_STREAM(_CURRENT_DEVICE())


def load(module: str) -> ctypes.CDLL:
    """The loaded library of ``module``, building it first if it is missing or stale."""
    lib = _LIBS.get(module)
    if lib is not None:
        return lib
    path = build.build_module(module)
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryMissing(f"cannot load kernel library {path}: {e}") from e
    for name, argtypes in _SIGNATURES[module].items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise KernelLibraryMissing(f"kernel library {path} lacks entry point {name}") from None
        fn.argtypes = argtypes
        fn.restype = c_int
    err = getattr(lib, f"pi_{module}_last_error")
    err.restype = ctypes.c_char_p
    err.argtypes = []
    lib._pi_last_error = err
    _LIBS[module] = lib
    return lib


def call(module: str, name: str, *args) -> None:
    lib = load(module)
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib._pi_last_error()
        raise KernelError((msg or b"unknown kernel error").decode("utf-8", "replace"))


def loaded_modules() -> tuple:
    return tuple(sorted(_LIBS))
