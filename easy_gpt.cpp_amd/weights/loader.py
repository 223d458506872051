"""Weights by tensor name, checked against what the model declares before anything is read.

The reference validates required keys and shapes before loading and reports
left-over keys afterwards (/root/reference/src/models/model_param_validation.cpp:84-218;
fixtures in /root/reference/test/model_param_validation_test.cpp:345-426).  Here one
error lists every missing tensor, every unexpected tensor and every wrong shape.

Stored dtypes: BF16 stays bfloat16, F32 stays float32, F16 and F64 become float32
(every float16 value is a float32 value, so nothing is lost), integer tables become
int32.  Parts cast 'compute' parameters to the engine's dtype when they take them:
that is the only rounding between the file and the device, as in the reference,
which decodes each element through float32 into the build's dtype
(/root/reference/src/models/loader.cpp:173-198).
"""
from __future__ import annotations

import json
import os
from typing import Iterable

import torch

from ..parts.spec import ParamSpec
from .safetensors_io import SafetensorsFile


class WeightsError(RuntimeError):
    """The weights file does not hold what the model declares."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def check_names_and_shapes(
    available: dict[str, tuple[int, ...]],
    specs: Iterable[ParamSpec],
    ignorable: Iterable[str] = (),
    where: str = "weights",
    allow_unexpected: bool = False,
) -> list[str]:
    """Compare the tensors on offer with the declared ones.  Raises one WeightsError that
    lists all problems; returns the names that were present but are not used (to warn about): the
    ignorable ones, and with allow_unexpected every other undeclared one, which the reference only
    warns about too (/root/reference/src/models/model_param_validation.cpp:198-218)."""
    specs = list(specs)
    declared = {s.name: s for s in specs}
    missing = [s.name for s in specs if s.name not in available]
    ignorable = set(ignorable)
    unexpected = [n for n in available if n not in declared and n not in ignorable and not allow_unexpected]
    ignored = [n for n in available if n not in declared and (n in ignorable or allow_unexpected)]
    wrong = []
    for name, spec in declared.items():
        if name in available:
            shape = tuple(available[name])
            if shape != tuple(spec.shape) and shape not in spec.alt_shapes:
                wrong.append((name, shape, tuple(spec.shape)))
    if missing or unexpected or wrong:
        lines = [f"{where} does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(
                f"  wrong shapes ({len(wrong)}): "
                + ", ".join(f"{n} is {list(got)}, expected {list(exp)}" for n, got, exp in wrong)
            )
        raise WeightsError("\n".join(lines), missing, unexpected, wrong)
    return ignored


_STORED_AS = {
    torch.bfloat16: torch.bfloat16,
    torch.float16: torch.float32,
    torch.float32: torch.float32,
    torch.float64: torch.float32,
    torch.int32: torch.int32,
    torch.int64: torch.int32,
}


class CheckedWeights:
    """The safetensors file(s) of a model folder whose names and shapes were checked; `get(name)` reads one tensor.

    A folder holds `model.safetensors` (all the reference reads, /root/reference/src/models/loader.cpp:45-63),
    or, for checkpoints stored in several files, `model.safetensors.index.json` whose "weight_map" names the
    file of every tensor."""

    INDEX = "model.safetensors.index.json"

    def __init__(self, model_dir: str, specs: Iterable[ParamSpec], ignorable: Iterable[str] = (),
                 allow_unexpected: bool = False):
        self.path = os.path.join(model_dir, "model.safetensors")
        self.files: list[SafetensorsFile] = []
        self._file_of: dict[str, SafetensorsFile] = {}
        index = os.path.join(model_dir, self.INDEX)
        try:
            if not os.path.isfile(self.path) and os.path.isfile(index):
                self.path = index
                self._open_shards(model_dir, index)
            else:
                f = SafetensorsFile(self.path)
                self.files.append(f)
                self._file_of = {n: f for n in f.names()}
            available = {n: f.shape(n) for n, f in self._file_of.items()}
            self.ignored = check_names_and_shapes(available, specs, ignorable, where=self.path,
                                                  allow_unexpected=allow_unexpected)
        except Exception:
            self.close()
            raise

    def _open_shards(self, model_dir: str, index: str) -> None:
        try:
            with open(index, "r", encoding="utf-8") as fh:
                weight_map = json.load(fh)["weight_map"]
            assert isinstance(weight_map, dict) and all(isinstance(v, str) for v in weight_map.values())
        except (OSError, ValueError, KeyError, TypeError, AssertionError) as e:
            raise WeightsError(f"{index}: not an index with a 'weight_map' of tensor name -> file ({e})") from e
        opened: dict[str, SafetensorsFile] = {}
        for name, rel in weight_map.items():
            if os.path.basename(rel) != rel:
                raise WeightsError(f"{index}: file '{rel}' of tensor '{name}' must lie in the model folder")
            if rel not in opened:
                opened[rel] = SafetensorsFile(os.path.join(model_dir, rel))
                self.files.append(opened[rel])
            if name not in opened[rel].entries:
                raise WeightsError(f"{index}: tensor '{name}' is not in '{rel}'")
            self._file_of[name] = opened[rel]
        # a tensor that a file holds but the index does not name is reported as unexpected by the check
        for rel, f in opened.items():
            for name in f.names():
                self._file_of.setdefault(name, f)

    def get(self, name: str) -> torch.Tensor:
        t = self._file_of[name].read(name)
        target = _STORED_AS[t.dtype]
        if t.dtype == torch.int64 and t.numel():
            if int(t.max()) > 2**31 - 1 or int(t.min()) < -(2**31):
                raise WeightsError(f"{self.path}: integer tensor '{name}' does not fit int32")
        return t if t.dtype == target else t.to(target)

    def close(self) -> None:
        for f in self.files:
            f.close()
        self.files = []
