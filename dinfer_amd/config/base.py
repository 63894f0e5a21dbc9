"""Typed reading of a model's config.json.

A configuration class lists the keys it reads as dataclass fields declared with
``key(type, ...)``. ``from_dict`` reads each key from the parsed JSON with a
type check and either a default or a "required" error that names the key.
Unknown keys are ignored: config.json files carry many that inference does not
need.
"""
from __future__ import annotations

import json
from dataclasses import MISSING, dataclass, field, fields
from pathlib import Path
from typing import Any


class ConfigError(ValueError):
    """A config.json that cannot be used: the message names the key and the offending value."""


_ACCEPTS = {int: (int,), float: (int, float), bool: (bool,), str: (str,)}


def key(typ: type, default: Any = MISSING, *, nullable: bool = False):
    """A dataclass field that is read from the config.json key of the same name."""
    meta = {"type": typ, "nullable": nullable}
    if default is MISSING:
        return field(metadata=meta)
    return field(default=default, metadata=meta)


def coerce(name: str, value: Any, typ: type) -> Any:
    if typ in (int, float) and isinstance(value, bool):
        raise ConfigError(f"config key {name!r} must be {typ.__name__}, got {value!r}")
    if typ is int and isinstance(value, float) and value == int(value):
        return int(value)
    if not isinstance(value, _ACCEPTS[typ]):
        raise ConfigError(f"config key {name!r} must be {typ.__name__}, got {value!r}")
    return typ(value)


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's configuration.

    Keys of a plain type are declared with ``key``; anything structured (a list,
    a value that may be a number or a list) is produced by ``extra_from_dict``
    and written back by ``extra_to_dict``.
    """

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        if not isinstance(d, dict):
            raise ConfigError("config.json must hold a JSON object")
        kw = {}
        for f in fields(cls):
            typ = f.metadata.get("type")
            if typ is None:
                continue
            if f.name not in d:
                if f.default is not MISSING:
                    continue
                raise ConfigError(f"config.json lacks the required key {f.name!r}")
            v = d[f.name]
            if v is None:
                if f.metadata.get("nullable"):
                    kw[f.name] = None
                    continue
                raise ConfigError(f"config key {f.name!r} must be {typ.__name__}, got null")
            kw[f.name] = coerce(f.name, v, typ)
        kw.update(cls.extra_from_dict(d))
        cfg = cls(**kw)
        cfg.check()
        return cfg

    @classmethod
    def extra_from_dict(cls, d: dict) -> dict:
        return {}

    def extra_to_dict(self) -> dict:
        return {}

    def check(self) -> None:
        """Raises ConfigError for values and options the engine does not implement."""

    @classmethod
    def from_json_file(cls, path: str | Path) -> "ModelConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def to_dict(self) -> dict:
        """The config.json content that reads back into an equal configuration."""
        out = {f.name: getattr(self, f.name) for f in fields(self) if f.metadata.get("type") is not None}
        out.update(self.extra_to_dict())
        return out
