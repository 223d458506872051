"""One registry from an architecture's name to its configuration class and model builder.

The reference picks its tensor-name builder by architecture / model_type and
throws std::invalid_argument naming both strings when neither is known
(/root/reference/src/models/layer_key_prefix.cpp:17-28,92-105; vectors in
/root/reference/test/layer_key_prefix_test.cpp:23-47).
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Any, Callable, Mapping

from .base import ConfigError, read_json


class UnknownArchitectureError(ConfigError):
    pass


@dataclass(frozen=True)
class Architecture:
    """What the framework needs to know of one architecture.

    name           the string in config.json's ``architectures[0]``
    model_types    values of ``model_type`` that also select it
    config_class   has ``from_dict(mapping, where) -> config`` and ``to_dict()``
    build_spec     ``config -> parts.ModelSpec``: the layers, their parts and the run order
    """

    name: str
    config_class: Any
    build_spec: Callable[[Any], Any]
    model_types: tuple[str, ...] = field(default_factory=tuple)


_BY_NAME: dict[str, Architecture] = {}
_BY_MODEL_TYPE: dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False) -> Architecture:
    if not replace and arch.name in _BY_NAME:
        raise ValueError(f"architecture '{arch.name}' is already registered")
    _BY_NAME[arch.name] = arch
    for mt in arch.model_types:
        _BY_MODEL_TYPE[mt.lower()] = arch
    return arch


def unregister_architecture(name: str) -> None:
    arch = _BY_NAME.pop(name, None)
    if arch is not None:
        for mt in arch.model_types:
            if _BY_MODEL_TYPE.get(mt.lower()) is arch:
                del _BY_MODEL_TYPE[mt.lower()]


def registered_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_BY_NAME)


def _ensure_builtin() -> None:
    # The built-in architectures register themselves on import.
    from .. import architectures  # noqa: F401


def resolve_architecture(config: Mapping[str, Any]) -> Architecture:
    """Architecture named by a config.json mapping: ``architectures[0]`` first, then ``model_type``."""
    _ensure_builtin()
    archs = config.get("architectures")
    name = archs[0] if isinstance(archs, list) and archs and isinstance(archs[0], str) else ""
    model_type = config.get("model_type") if isinstance(config.get("model_type"), str) else ""
    if name in _BY_NAME:
        return _BY_NAME[name]
    if model_type.lower() in _BY_MODEL_TYPE:
        return _BY_MODEL_TYPE[model_type.lower()]
    raise UnknownArchitectureError(
        f"unsupported model: architecture='{name}', model_type='{model_type}' "
        f"(registered: {', '.join(sorted(_BY_NAME)) or 'none'})"
    )


def load_model_config(model_dir: str):
    """Read ``model_dir/config.json`` -> (Architecture, typed config)."""
    path = os.path.join(model_dir, "config.json")
    data = read_json(path)
    arch = resolve_architecture(data)
    return arch, arch.config_class.from_dict(data, where=path)
