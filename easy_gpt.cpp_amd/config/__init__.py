from .base import ConfigError, KeyReader, read_json
from .qwen2 import Qwen2Config
from .registry import (
    Architecture,
    UnknownArchitectureError,
    load_model_config,
    register_architecture,
    registered_architectures,
    resolve_architecture,
    unregister_architecture,
)

__all__ = [
    "Architecture",
    "ConfigError",
    "KeyReader",
    "Qwen2Config",
    "UnknownArchitectureError",
    "load_model_config",
    "read_json",
    "register_architecture",
    "registered_architectures",
    "resolve_architecture",
    "unregister_architecture",
]
