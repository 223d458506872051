"""Typed reading of config.json keys.

Every value a model needs comes from a key of its config.json; a key that is
absent and has no documented default, or that has the wrong type or range, is
reported by name.
"""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Mapping

_REQUIRED = object()


class ConfigError(ValueError):
    """A config.json key is missing, of the wrong type or out of range."""


def read_json(path: str) -> dict:
    if not os.path.isfile(path):
        raise ConfigError(f"config file not found: {path}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            data = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from e
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return data


class KeyReader:
    """Reads keys of one JSON object with type checks; remembers which keys were read."""

    def __init__(self, data: Mapping[str, Any], where: str = "config.json"):
        self.data = data
        self.where = where
        self.seen: set[str] = set()

    def _get(self, key: str, default: Any) -> Any:
        self.seen.add(key)
        if key not in self.data or self.data[key] is None:
            if default is _REQUIRED:
                raise ConfigError(f"{self.where}: required key '{key}' is missing")
            return default
        return self.data[key]

    def integer(self, key: str, default: Any = _REQUIRED, minimum: int | None = None) -> int | None:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v.is_integer():
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: key '{key}' must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: key '{key}' must be >= {minimum}, got {v}")
        return v

    def number(self, key: str, default: Any = _REQUIRED, positive: bool = False) -> float | None:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key '{key}' must be a number, got {v!r}")
        v = float(v)
        if positive and not v > 0.0:
            raise ConfigError(f"{self.where}: key '{key}' must be > 0, got {v}")
        return v

    def boolean(self, key: str, default: Any = _REQUIRED) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: key '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _REQUIRED, check: Callable[[str], bool] | None = None) -> str:
        v = self._get(key, default)
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: key '{key}' must be a string, got {v!r}")
        if check is not None and not check(v):
            raise ConfigError(f"{self.where}: key '{key}' has unsupported value {v!r}")
        return v

    def token_id(self, key: str) -> int:
        """A token id, -1 when absent; a list (several end tokens) gives its first entry."""
        v = self._get(key, -1)
        if isinstance(v, list):
            v = v[0] if v else -1
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{self.where}: key '{key}' must be an integer token id, got {v!r}")
        return v
