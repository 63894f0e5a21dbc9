"""The one registry from an architecture's name to its model.

config.json names the architecture in ``architectures[0]``; the entry gives the
configuration class that reads the file and the function that turns a
configuration into a ``ModelSpec`` (layer parts, run order, weight names).

The reference has no such table: it picks the model at compile time by a cargo
feature (bins/dinfer/src/main.rs:6-18,153-178).
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Callable

from .base import ConfigError, ModelConfig


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable  # (config) -> parts.spec.ModelSpec


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, build_spec: Callable) -> Architecture:
    arch = Architecture(name, config_class, build_spec)
    _ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def _load_builtin() -> None:
    from .. import models  # noqa: F401  (registers the built-in architectures)


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"unknown architecture {name!r}; known: {sorted(_ARCHITECTURES)}") from None


def architecture_of(config_dict: dict) -> Architecture:
    archs = config_dict.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json must name the model in 'architectures' (a non-empty list of strings)")
    return get_architecture(archs[0])


def load_config(model_dir: str | Path) -> tuple[Architecture, ModelConfig]:
    """Reads DIR/config.json and returns (architecture entry, typed configuration)."""
    path = Path(model_dir) / "config.json"
    if not path.exists():
        raise ConfigError(f"{path} does not exist")
    try:
        d = json.loads(path.read_text())
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from e
    arch = architecture_of(d)
    return arch, arch.config_class.from_dict(d)
