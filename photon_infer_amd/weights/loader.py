"""Name-based weight loading with one error that lists everything wrong.

The reference reads a positional blob and hands slices to setters
(src/io/checkpoint.cpp:106-317); shape problems surface one at a time from each
setter (include/photon/ops/matmul.hpp:89-109).  Here the model says which tensors it
expects (name, shape, role); the folder is compared against that list as a whole and
a single ``WeightError`` names every missing tensor, every unexpected tensor and
every tensor whose shape differs.

Storage policy: floating tensors are kept in bfloat16 unless the file stores them in
32-bit (then they stay 32-bit); 16-bit float becomes bfloat16; integer tables become
int32.  In the float32 compute mode every floating tensor is widened to float32.
"""
from __future__ import annotations

import fnmatch
from dataclasses import dataclass
from typing import Dict, Iterable, Mapping, Sequence, Tuple

import torch

from ..errors import WeightError
from .safetensors_io import SafetensorsFile, open_model_files


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part expects.

    ``role`` drives random initialisation only: "matrix" and "table" are drawn from
    N(0, std), "norm" follows the norm rule (ones or U(0.5, 1.5)), "int_table" holds
    integers.
    """

    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"

    def with_prefix(self, prefix: str) -> "TensorSpec":
        return TensorSpec(prefix + self.name, self.shape, self.role)


def storage_dtype(stored: torch.dtype, compute_dtype: torch.dtype) -> torch.dtype:
    """The dtype a tensor stored as ``stored`` is kept in under ``compute_dtype``."""
    if not stored.is_floating_point:
        return torch.int32
    if compute_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def check_tensors(
    expected: Mapping[str, TensorSpec],
    found: Mapping[str, Tuple[int, ...]],
    ignorable: Sequence[str] = (),
    where: str = "model",
) -> None:
    """Raise one WeightError listing missing, unexpected and wrongly shaped tensors."""
    missing = [n for n in expected if n not in found]
    unexpected = [
        n for n in found if n not in expected and not any(fnmatch.fnmatchcase(n, p) for p in ignorable)
    ]
    wrong = [
        (n, tuple(expected[n].shape), tuple(found[n]))
        for n in expected
        if n in found and tuple(found[n]) != tuple(expected[n].shape)
    ]
    if not (missing or unexpected or wrong):
        return
    lines = [f"{where}: weights do not match the model"]
    if missing:
        lines.append(f"  missing ({len(missing)}):")
        lines += [f"    {n}  expected shape {list(expected[n].shape)}" for n in sorted(missing)]
    if unexpected:
        lines.append(f"  unexpected ({len(unexpected)}):")
        lines += [f"    {n}  shape {list(found[n])}" for n in sorted(unexpected)]
    if wrong:
        lines.append(f"  wrong shape ({len(wrong)}):")
        lines += [f"    {n}  expected {list(e)}, file has {list(f)}" for n, e, f in sorted(wrong)]
    err = WeightError("\n".join(lines))
    err.missing = sorted(missing)
    err.unexpected = sorted(unexpected)
    err.wrong_shape = sorted(wrong)
    raise err


def load_model_tensors(
    model_dir: str,
    expected: Iterable[TensorSpec],
    compute_dtype: torch.dtype,
    device: torch.device | str,
    ignorable: Sequence[str] = (),
) -> Dict[str, torch.Tensor]:
    """Load exactly the expected tensors of ``model_dir`` onto ``device``."""
    exp = {s.name: s for s in expected}
    files = open_model_files(model_dir)
    try:
        owner: Dict[str, SafetensorsFile] = {}
        for f in files:
            for n in f.names():
                owner[n] = f
        check_tensors(exp, {n: owner[n].entries[n].shape for n in owner}, ignorable, model_dir)
        out: Dict[str, torch.Tensor] = {}
        for name in exp:
            t = owner[name].read(name)
            out[name] = t.to(device=device, dtype=storage_dtype(t.dtype, compute_dtype)).contiguous()
        return out
    finally:
        for f in files:
            f.close()
