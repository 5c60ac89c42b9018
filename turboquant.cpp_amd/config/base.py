"""Typed reading of a model folder's ``config.json``.

The reference never reads ``config.json`` (its safetensors loader sniffs shapes,
/root/reference/src/engine/tq_model.c:949-1223, and its GGUF loader reads
metadata keys, tq_model.c:2867-2905).  Here every size and constant of a model
comes from the keys of its own ``config.json``; a key that gives a size has no
default in code and its absence is an error.
"""
from __future__ import annotations

import json
import os
from typing import Any, Iterable, Sequence


class ConfigError(ValueError):
    """A config.json that is missing, malformed or inconsistent."""


_MISSING = object()


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in model folder {model_dir!r}")
    try:
        with open(path, "r", encoding="utf-8") as f:
            data = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from e
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return data


class KeyReader:
    """Reads typed keys of one JSON object and remembers which were used."""

    def __init__(self, data: dict, where: str = "config.json"):
        self.data = data
        self.where = where
        self.used: set[str] = set()

    def _get(self, key: str, default: Any = _MISSING) -> Any:
        self.used.add(key)
        if key in self.data and self.data[key] is not None:
            return self.data[key]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key {key!r} is missing")
        return default

    def integer(self, key: str, default: Any = _MISSING, minimum: int | None = None) -> int:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: key {key!r} must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: key {key!r} must be >= {minimum}, got {v}")
        return v

    def optional_integer(self, key: str) -> int | None:
        self.used.add(key)
        if self.data.get(key) is None:
            return None
        return self.integer(key)

    def number(self, key: str, default: Any = _MISSING) -> float:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key {key!r} must be a number, got {v!r}")
        return float(v)

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: key {key!r} must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING) -> str:
        v = self._get(key, default)
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: key {key!r} must be a string, got {v!r}")
        return v

    def integer_list(self, key: str, default: Any = _MISSING) -> list[int]:
        v = self._get(key, default)
        if isinstance(v, int) and not isinstance(v, bool):
            return [v]
        if not isinstance(v, (list, tuple)) or any(isinstance(i, bool) or not isinstance(i, int) for i in v):
            raise ConfigError(f"{self.where}: key {key!r} must be a list of integers, got {v!r}")
        return list(v)


def architecture_name(data: dict) -> str:
    """The registry key of a config.json: the first entry of ``architectures``."""
    archs = data.get("architectures")
    if isinstance(archs, str):
        return archs
    if not isinstance(archs, Sequence) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: key 'architectures' must name the model class, e.g. [\"Qwen2MoeForCausalLM\"]")
    return archs[0]


def require(cond: bool, message: str) -> None:
    if not cond:
        raise ConfigError("config.json: " + message)


def flat_items(obj: Any, names: Iterable[str]) -> dict:
    return {n: getattr(obj, n) for n in names}
