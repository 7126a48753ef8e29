"""The sampling entry point that allocates nothing (``pi_sample_static``), called through ctypes
as a caller without an allocator would, against ``pi_sample`` with a workspace."""
from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _library() -> ctypes.CDLL:
    from photon_infer_amd.ops import build

    lib = ctypes.CDLL(build.build_module("core"))
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    lib.pi_sample.argtypes = [P, P, L, P, P, I, I, P, L, P]
    lib.pi_sample_static.argtypes = [P, P, L, P, P, I, I, P]
    lib.pi_sample_chunks.argtypes = [I]
    for fn in (lib.pi_sample, lib.pi_sample_static, lib.pi_sample_chunks):
        fn.restype = I
    lib.pi_core_last_error.restype = ctypes.c_char_p
    return lib


def _case(M: int, V: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(M, V, generator=g) * 3.0).to(DEV)
    temps = torch.tensor([0.0 if m % 3 == 0 else 0.5 + 0.25 * m for m in range(M)], dtype=torch.float32, device=DEV)
    draws = torch.rand(M, generator=g).to(DEV)
    return logits, temps, draws


def test_sampling_without_allocation_matches_the_workspace_entry_point():
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    # two calls in a row on the library's one array, the second smaller in rows and in row length,
    # then a short vocabulary that needs no records at all
    for M, V, seed in ((7, 128256, 1), (3, 50021, 2), (5, 1001, 3)):
        logits, temps, draws = _case(M, V, seed)
        chunks = lib.pi_sample_chunks(V)
        ws = torch.empty(max(1, M * chunks * 4), dtype=torch.float32, device=DEV)
        want = torch.full((M,), -1, dtype=torch.int32, device=DEV)
        got = torch.full((M,), -2, dtype=torch.int32, device=DEV)
        assert lib.pi_sample(want.data_ptr(), logits.data_ptr(), V, temps.data_ptr(), draws.data_ptr(), M, V,
                             ws.data_ptr(), ws.numel(), stream) == 0, lib.pi_core_last_error()
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        assert lib.pi_sample_static(got.data_ptr(), logits.data_ptr(), V, temps.data_ptr(), draws.data_ptr(), M, V,
                                    stream) == 0, lib.pi_core_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert got.tolist() == want.tolist(), (M, V)
        assert all(0 <= t < V for t in got.tolist())
        # greedy rows are the arg max
        assert [got[m].item() for m in range(0, M, 3)] == [int(logits[m].argmax()) for m in range(0, M, 3)]


def test_sampling_without_allocation_refuses_what_its_array_cannot_hold():
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    V = 140000                      # 64 chunks a row: the array holds 256 rows
    M = 257
    logits = torch.zeros((M, V), dtype=torch.float32, device=DEV)
    out = torch.full((M,), -7, dtype=torch.int32, device=DEV)
    rc = lib.pi_sample_static(out.data_ptr(), logits.data_ptr(), V, None, None, M, V, stream)
    assert rc != 0
    assert b"at most 256 rows" in lib.pi_core_last_error()
    torch.cuda.synchronize()
    assert out.tolist() == [-7] * M            # nothing ran
    rc = lib.pi_sample_static(out.data_ptr(), logits.data_ptr(), V, None, None, 256, V, stream)
    assert rc == 0, lib.pi_core_last_error()
    torch.cuda.synchronize()
    assert out.tolist() == [0] * 256 + [-7]
