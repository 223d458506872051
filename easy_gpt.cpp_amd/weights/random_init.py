"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and a seed.

Distributions: matrices, embeddings and biases ~ N(0, 0.02); norm scales ~ 1 + N(0, 0.02).
Each tensor is drawn from its own generator keyed by (seed, tensor name), so the
values do not depend on the order in which tensors are made.  (The reference only
has unseeded uniform constructors that nothing uses, /root/reference/src/models/linear.cpp:15-24.)
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Mapping

import torch

from ..config.registry import resolve_architecture
from ..parts.model import build_model
from ..parts.spec import ParamSpec
from .safetensors_io import write_safetensors

_STD = 0.02


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & (2**63 - 1))
    return g


def random_tensor(spec: ParamSpec, seed: int, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    g = _generator(seed, spec.name)
    if spec.role == "int_table":
        return torch.randint(0, 2**15, spec.shape, generator=g, dtype=torch.int32)
    t = torch.randn(spec.shape, generator=g, dtype=torch.float32) * _STD
    if spec.role == "norm_scale":
        t = t + 1.0
    if spec.dtype == "float32":
        return t
    return t.to(dtype)


def random_tensors(specs, seed: int, dtype: torch.dtype = torch.float32) -> dict[str, torch.Tensor]:
    return {s.name: random_tensor(s, seed, dtype) for s in specs}


def write_random_model(
    model_dir: str, config: Mapping[str, Any], seed: int, dtype: torch.dtype = torch.float32
) -> str:
    """Write `model_dir/config.json` and `model_dir/model.safetensors` for the architecture that
    `config` (a config.json mapping) names.  Returns model_dir."""
    arch = resolve_architecture(config)
    typed = arch.config_class.from_dict(config, where="config")
    model = build_model(arch.build_spec(typed))
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(dict(config), f, indent=1)
    tensors = random_tensors(model.param_specs(), seed, dtype)
    write_safetensors(
        os.path.join(model_dir, "model.safetensors"), tensors, metadata={"format": "pt", "seed": str(seed)}
    )
    return model_dir
