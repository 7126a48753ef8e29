"""Reading and writing the safetensors container (no third-party reader).

Layout: 8 bytes little-endian header length N, N bytes of JSON
``{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}``,
then the raw little-endian payload; offsets are relative to the payload start.

The reference maps its weight file with mmap and copies slices out of it
(src/io/checkpoint.cpp:25-68,106-317) but does not detect a truncated file; here every
tensor's byte range is checked against the file before anything is read.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, Mapping, Tuple

import torch

from ..errors import ErrorCode, FileFormatError

# safetensors dtype tag -> (torch dtype, bytes per element)
_DTYPES = {
    "F64": (torch.float64, 8),
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_TAG_OF = {v[0]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int  # absolute file offsets
    end: int


class SafetensorsFile:
    """One mapped .safetensors file; tensors are views of the mapping until copied."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise FileFormatError(f"weight file '{path}' does not exist", ErrorCode.FILE_NOT_FOUND)
        size = os.path.getsize(path)
        if size < 8:
            raise FileFormatError(f"{path}: too small to be a safetensors file ({size} bytes)")
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise FileFormatError(f"{path}: header length {hlen} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except ValueError as e:
            raise FileFormatError(f"{path}: header is not valid JSON: {e}") from e
        if not isinstance(header, dict):
            raise FileFormatError(f"{path}: header must be a JSON object")
        self.metadata = header.pop("__metadata__", None) or {}
        base = 8 + hlen
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            try:
                tag, shape, (b, e) = info["dtype"], tuple(int(s) for s in info["shape"]), info["data_offsets"]
            except (KeyError, TypeError, ValueError) as ex:
                raise FileFormatError(f"{path}: malformed entry for tensor '{name}': {ex}") from ex
            if tag not in _DTYPES:
                raise FileFormatError(
                    f"{path}: tensor '{name}' has unsupported dtype '{tag}'", ErrorCode.INVALID_DTYPE
                )
            dtype, width = _DTYPES[tag]
            count = 1
            for s in shape:
                count *= s
            if b < 0 or e < b or e - b != count * width:
                raise FileFormatError(
                    f"{path}: tensor '{name}' {tag}{list(shape)} needs {count * width} bytes "
                    f"but its offsets give {e - b}"
                )
            if base + e > size:
                raise FileFormatError(
                    f"{path}: tensor '{name}' ends at byte {base + e} but the file has {size} (truncated?)"
                )
            self.entries[name] = TensorEntry(name, dtype, shape, base + b, base + e)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor that owns its memory (copied out of the mapping)."""
        e = self.entries[name]
        n = e.end - e.begin
        if n == 0:
            return torch.empty(e.shape, dtype=e.dtype)
        buf = bytearray(self._map[e.begin : e.end])  # one copy; frees us from the mapping's lifetime
        return torch.frombuffer(buf, dtype=e.dtype).reshape(e.shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] | None = None) -> None:
    """Write CPU tensors to ``path``; entries are laid out in sorted-name order."""
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _TAG_OF:
            raise FileFormatError(f"cannot store tensor '{name}' of dtype {t.dtype}", ErrorCode.INVALID_DTYPE)
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAG_OF[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            # view as bytes without going through numpy (bfloat16 has no numpy dtype)
            f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)


def open_model_files(model_dir: str) -> list:
    """The weight files of a model folder: ``model.safetensors`` or the shards that
    ``model.safetensors.index.json`` names."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    if os.path.isfile(index):
        try:
            with open(index, "r", encoding="utf-8") as f:
                weight_map = json.load(f)["weight_map"]
        except (OSError, ValueError, KeyError) as e:
            raise FileFormatError(f"{index}: cannot read weight_map: {e}") from e
        return [SafetensorsFile(os.path.join(model_dir, s)) for s in sorted(set(weight_map.values()))]
    raise FileFormatError(
        f"model folder '{model_dir}' has neither model.safetensors nor model.safetensors.index.json",
        ErrorCode.FILE_NOT_FOUND,
    )
