"""One registry from an architecture's name to its configuration class and model plan.

The reference picks its model type with ``strstr`` on the GGUF architecture string
(/root/reference/src/engine/tq_model.c:3031-3056); here the key is the exact class
name in ``config.json`` and an unknown name is an error that lists the known ones
(error style of /root/reference/bindings/python/quantcpp/__init__.py:199-205).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

from .base import ConfigError, architecture_name, read_config_json
from .plan import ModelPlan


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_json: Callable[[dict], Any]      # dict of config.json -> typed configuration
    plan: Callable[[Any], ModelPlan]             # typed configuration -> model plan
    config_to_json: Callable[[Any], dict]        # typed configuration -> dict for config.json
    random_tensors: Callable[..., Any] | None = None   # (config, seed, ...) -> iterator of (name, tensor)


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> None:
    if arch.name in _ARCHITECTURES:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch


def known_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def lookup_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture {name!r}; known: {', '.join(known_architectures()) or '(none)'}"
        ) from None


def config_from_dict(data: dict):
    arch = lookup_architecture(architecture_name(data))
    return arch, arch.config_from_json(data)


def config_from_dir(model_dir: str):
    """Reads ``config.json`` of a model folder; returns (architecture entry, typed configuration)."""
    return config_from_dict(read_config_json(model_dir))
