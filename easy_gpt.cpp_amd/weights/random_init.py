"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and a seed.

Distributions by a tensor's role (`ParamSpec.role`): matrices, embeddings and biases ~ N(0, 0.02); norm scales
~ 1 + N(0, 0.02); integer tables uniform.  `register_role` adds a role with a distribution of its own.
Each tensor has a key made of (seed, tensor name), and element i of it is a function of (key, i) alone, computed
with integer operations: the values do not depend on the order in which tensors are made nor on the device that
draws them (a GPU draws a large model's tensors in seconds, the CPU draws the same ones).  The normal distribution is
approximated by a sum of eight 16-bit uniform integers (Irwin-Hall: the right mean and variance, no value beyond 4.9
standard deviations), because integer sums are the same bits everywhere and logarithms and cosines are not.  A role
added with `register_role` draws as it likes from a torch.Generator seeded with the key (such values do depend on the
device).  `RandomWeights` hands the same tensors to a model without a file in between.  (The reference only has
unseeded uniform constructors that nothing uses, /root/reference/src/models/linear.cpp:15-24.)
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Callable, Mapping

import torch

from ..config.registry import resolve_architecture
from ..parts.model import build_model
from ..parts.spec import ParamSpec
from .safetensors_io import write_safetensors

_STD = 0.02


def _generator(seed: int, name: str, device: str = "cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & (2**63 - 1))
    return g


# splitmix64 on int64 tensors (two's complement wraps the same way on every device; shifts are made logical by a mask)
_GOLD, _C1, _C2 = 0x9E3779B97F4A7C15, 0xBF58476D1CE4E5B9, 0x94D049BB133111EB
_CHUNK = 1 << 24          # elements drawn at a time: bounds the temporaries of a large tensor


def _signed(c: int) -> int:
    return c - (1 << 64) if c >= 1 << 63 else c


def _lsr(z: torch.Tensor, k: int) -> torch.Tensor:
    return (z >> k) & ((1 << (64 - k)) - 1)


def _mix(z: torch.Tensor) -> torch.Tensor:
    z = z + _signed(_GOLD)
    z = (z ^ _lsr(z, 30)) * _signed(_C1)
    z = (z ^ _lsr(z, 27)) * _signed(_C2)
    return z ^ _lsr(z, 31)


def _hashes(key: int, first: int, count: int, device) -> tuple[torch.Tensor, torch.Tensor]:
    """Two 64-bit hashes of (key, i) for i in [first, first + count)."""
    i = torch.arange(first, first + count, dtype=torch.int64, device=device)
    h1 = _mix(i * _signed(_GOLD) + _signed(key & ((1 << 64) - 1)))
    return h1, _mix(h1 ^ _signed(_C1))


def _sum_of_uniforms(h1: torch.Tensor, h2: torch.Tensor) -> torch.Tensor:
    """The sum of the eight 16-bit fields of two 64-bit hashes (fields added two at a time inside the words)."""
    even = 0x0000FFFF0000FFFF
    pairs = (h1 & even) + ((h1 >> 16) & even) + (h2 & even) + ((h2 >> 16) & even)      # two sums of four fields
    return (pairs & 0xFFFFFFFF) + ((pairs >> 32) & 0xFFFFFFFF)


# eight uniform integers on [0, 65535]: mean 8 * 65535 / 2, variance 8 * (65536^2 - 1) / 12
_SUM_MEAN = 8 * 65535 / 2
_SUM_STD = (8 * (65536.0 ** 2 - 1) / 12) ** 0.5


def _counter_normal(shape, key: int, device, std: float, mean: float = 0.0) -> torch.Tensor:
    n = 1
    for d in shape:
        n *= int(d)
    out = torch.empty(n, dtype=torch.float32, device=device)
    scale = torch.tensor(std / _SUM_STD, dtype=torch.float32).item()      # the float32 constant, the same everywhere
    for first in range(0, n, _CHUNK):
        count = min(_CHUNK, n - first)
        total = _sum_of_uniforms(*_hashes(key, first, count, device))
        v = (total.to(torch.float32) - _SUM_MEAN) * scale                 # an exact difference, then one rounding
        out[first : first + count] = v + mean if mean else v
    return out.view(tuple(shape))


def _normal(shape, g, device):
    return _counter_normal(shape, g.initial_seed(), device, _STD)


def _norm_scale(shape, g, device):
    return _counter_normal(shape, g.initial_seed(), device, _STD, 1.0)


def _int_table(shape, g, device):
    n = 1
    for d in shape:
        n *= int(d)
    h1, _ = _hashes(g.initial_seed(), 0, n, device)
    return (h1 & 0x7FFF).to(torch.int32).view(tuple(shape))


# role -> draw(shape, generator, device): float32 (or, for tensors kept as integers, int32) values on `device`.  The
# generator is seeded with the tensor's key; the built-in roles take only that key from it.
ROLES: dict[str, Callable[..., torch.Tensor]] = {
    "matrix": _normal,
    "embedding": _normal,
    "bias": _normal,
    "norm_scale": _norm_scale,
    "int_table": _int_table,
}


def register_role(role: str, draw: Callable[..., torch.Tensor], replace: bool = False) -> None:
    """Add a way to draw random weights: `draw(shape, generator, device)` returns the float32 values of a tensor
    whose `ParamSpec.role` is `role` (say, decays within (0, 1)).  Parts of another architecture use it for tensors
    that none of the built-in distributions suits."""
    if role in ROLES and not replace:
        raise ValueError(f"role '{role}' is already registered")
    ROLES[role] = draw


def _drawing_device(device) -> str:
    """Where tensors are drawn when the caller does not say: a GPU if there is one (the values are the same)."""
    if device is not None:
        return device
    return "cuda" if torch.cuda.is_available() else "cpu"


def random_tensor(spec: ParamSpec, seed: int, dtype: torch.dtype = torch.float32, device: str | None = None,
                  to_host: bool = True) -> torch.Tensor:
    """The tensor that `spec` declares, drawn on `device` and returned in host memory (or left where it was drawn)."""
    device = _drawing_device(device)
    if spec.role not in ROLES:
        raise KeyError(f"tensor '{spec.name}' has the role '{spec.role}', which has no distribution "
                       f"(registered: {', '.join(sorted(ROLES))}; see register_role)")
    t = ROLES[spec.role](tuple(spec.shape), _generator(seed, spec.name, device), device)
    if spec.dtype == "compute" and t.is_floating_point():
        t = t.to(dtype)
    return t.cpu() if to_host else t


def random_tensors(specs, seed: int, dtype: torch.dtype = torch.float32, device: str | None = None) -> dict[str, torch.Tensor]:
    return {s.name: random_tensor(s, seed, dtype, device) for s in specs}


class RandomWeights:
    """The tensors of `write_random_model` without the file: `get(name)` draws the declared tensor on `device` and
    leaves it there, for `Model.load`.  For models whose file would be tens of gigabytes (the values are the file's)."""

    def __init__(self, specs, seed: int, dtype: torch.dtype = torch.float32, device: str | None = None):
        self.specs = {s.name: s for s in specs}
        self.seed, self.dtype, self.device = int(seed), dtype, _drawing_device(device)

    def get(self, name: str) -> torch.Tensor:
        if name not in self.specs:
            raise KeyError(f"the model declares no tensor '{name}'")
        return random_tensor(self.specs[name], self.seed, self.dtype, self.device, to_host=False)


def write_random_model(
    model_dir: str, config: Mapping[str, Any], seed: int, dtype: torch.dtype = torch.float32, device: str | None = None
) -> str:
    """Write `model_dir/config.json` and `model_dir/model.safetensors` for the architecture that
    `config` (a config.json mapping) names, its tensors drawn on `device` (default: a GPU if there is one, else the
    CPU; the file is the same either way).  Returns model_dir."""
    arch = resolve_architecture(config)
    typed = arch.config_class.from_dict(config, where="config")
    model = build_model(arch.build_spec(typed))
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(dict(config), f, indent=1)
    tensors = random_tensors(model.param_specs(), seed, dtype, device)
    write_safetensors(
        os.path.join(model_dir, "model.safetensors"), tensors, metadata={"format": "pt", "seed": str(seed)}
    )
    return model_dir
