"""Reading and writing of a single ``model.safetensors`` file.

Format (as the reference parses it, /root/reference/src/models/loader.cpp:213-252,
298-310): an unsigned 64-bit little-endian header length, a JSON header mapping
each tensor name to {dtype, shape, data_offsets}, then the raw data.  The key
``__metadata__`` is skipped.  Offsets are relative to the end of the header, must
be ordered, lie inside the file and span numel * width bytes.
"""
from __future__ import annotations

import json
import mmap
import warnings
import os
import struct
from dataclasses import dataclass

import torch


class SafetensorsError(RuntimeError):
    pass


# name in the file -> (torch dtype, bytes per element)
_DTYPES = {
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F32": (torch.float32, 4),
    "F64": (torch.float64, 8),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: tuple[int, ...]
    begin: int
    end: int


class SafetensorsFile:
    """A memory-mapped safetensors file: header parsed and checked at open, data read on demand."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise SafetensorsError(f"weights file not found: {path}")
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too small to hold a safetensors header")
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._mm[:8])
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._mm[8 : 8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from e
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self._data_start = 8 + hlen
        data_size = size - self._data_start
        self.entries: dict[str, TensorEntry] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            self.entries[name] = self._check_entry(name, info, data_size)

    def _check_entry(self, name: str, info, data_size: int) -> TensorEntry:
        p = self.path
        if not isinstance(info, dict):
            raise SafetensorsError(f"{p}: entry '{name}' is not an object")
        dtype = info.get("dtype")
        if dtype not in _DTYPES:
            raise SafetensorsError(f"{p}: tensor '{name}' has unsupported dtype {dtype!r}")
        shape = info.get("shape")
        if not isinstance(shape, list) or any(isinstance(s, bool) or not isinstance(s, int) or s < 0 for s in shape):
            raise SafetensorsError(f"{p}: tensor '{name}' has an invalid shape {shape!r}")
        offs = info.get("data_offsets")
        if (
            not isinstance(offs, list)
            or len(offs) != 2
            or any(isinstance(o, bool) or not isinstance(o, int) for o in offs)
        ):
            raise SafetensorsError(f"{p}: tensor '{name}' has invalid data_offsets {offs!r}")
        begin, end = offs
        if begin < 0 or end < begin or end > data_size:
            raise SafetensorsError(
                f"{p}: tensor '{name}' data_offsets [{begin}, {end}) lie outside the data section ({data_size} bytes)"
            )
        numel = 1
        for s in shape:
            numel *= s
        width = _DTYPES[dtype][1]
        if end - begin != numel * width:
            raise SafetensorsError(
                f"{p}: tensor '{name}' spans {end - begin} bytes but shape {shape} of {dtype} needs {numel * width}"
            )
        return TensorEntry(name, dtype, tuple(shape), begin, end)

    def names(self) -> list[str]:
        return list(self.entries)

    def shape(self, name: str) -> tuple[int, ...]:
        return self.entries[name].shape

    def read(self, name: str) -> torch.Tensor:
        """A copy of tensor `name` in the dtype it is stored in."""
        if name not in self.entries:
            raise KeyError(f"{self.path}: no tensor named '{name}'")
        e = self.entries[name]
        dtype, _ = _DTYPES[e.dtype]
        if e.end == e.begin:
            return torch.empty(e.shape, dtype=dtype)
        # one copy, from the mapped file into the tensor (the view itself must not outlive the mapping)
        view = memoryview(self._mm)[self._data_start + e.begin : self._data_start + e.end]
        try:
            with warnings.catch_warnings():
                warnings.simplefilter("ignore", UserWarning)          # "the given buffer is not writable"
                return torch.frombuffer(view, dtype=dtype).reshape(e.shape).clone()
        finally:
            view.release()

    def close(self) -> None:
        try:
            self._mm.close()
        finally:
            self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict[str, str] | None = None) -> None:
    """Write `tensors` (CPU, any of the supported dtypes) as one safetensors file."""
    header: dict = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot write tensor '{name}' of dtype {t.dtype}")
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    hjson = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for raw in blobs:
            f.write(raw)
