"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and a seed.

Distributions by a tensor's role (`ParamSpec.role`): matrices, embeddings and biases ~ N(0, 0.02); norm scales
~ 1 + N(0, 0.02); integer tables uniform.  `register_role` adds a role with a distribution of its own.
Each tensor is drawn from its own generator keyed by (seed, tensor name), so the
values do not depend on the order in which tensors are made; they do depend on the
device that draws them (the CPU unless asked otherwise: a GPU draws a large model's
tensors in seconds, with other values for the same seed).  (The reference only
has unseeded uniform constructors that nothing uses, /root/reference/src/models/linear.cpp:15-24.)
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


def _normal(shape, g, device):
    return torch.randn(shape, generator=g, dtype=torch.float32, device=device) * _STD


# role -> draw(shape, generator, device): float32 (or, for tensors kept as integers, int32) values on `device`
ROLES: dict[str, Callable[..., torch.Tensor]] = {
    "matrix": _normal,
    "embedding": _normal,
    "bias": _normal,
    "norm_scale": lambda shape, g, device: _normal(shape, g, device) + 1.0,
    "int_table": lambda shape, g, device: torch.randint(0, 2**15, shape, generator=g, dtype=torch.int32, device=device),
}


def register_role(role: str, draw: Callable[..., torch.Tensor], replace: bool = False) -> None:
    """Add a way to draw random weights: `draw(shape, generator, device)` returns the float32 values of a tensor
    whose `ParamSpec.role` is `role` (say, decays within (0, 1)).  Parts of another architecture use it for tensors
    that none of the built-in distributions suits."""
    if role in ROLES and not replace:
        raise ValueError(f"role '{role}' is already registered")
    ROLES[role] = draw


def random_tensor(spec: ParamSpec, seed: int, dtype: torch.dtype = torch.float32, device: str = "cpu") -> torch.Tensor:
    """The tensor that `spec` declares, drawn on `device` and returned in host memory."""
    if spec.role not in ROLES:
        raise KeyError(f"tensor '{spec.name}' has the role '{spec.role}', which has no distribution "
                       f"(registered: {', '.join(sorted(ROLES))}; see register_role)")
    t = ROLES[spec.role](tuple(spec.shape), _generator(seed, spec.name, device), device)
    if spec.dtype != "compute" or not t.is_floating_point():
        return t.cpu()
    return t.to(dtype).cpu()


def random_tensors(specs, seed: int, dtype: torch.dtype = torch.float32, device: str = "cpu") -> dict[str, torch.Tensor]:
    return {s.name: random_tensor(s, seed, dtype, device) for s in specs}


def write_random_model(
    model_dir: str, config: Mapping[str, Any], seed: int, dtype: torch.dtype = torch.float32, device: str = "cpu"
) -> str:
    """Write `model_dir/config.json` and `model_dir/model.safetensors` for the architecture that
    `config` (a config.json mapping) names, its tensors drawn on `device`.  Returns model_dir."""
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
