"""Typed configurations read from config.json, and the architecture registry.

An architecture is registered under the name that config.json carries in
`architectures[0]`.  Its entry holds the configuration class that parses the
file's keys and the function that turns a configuration into a `ModelSpec`
(the list of parts, layer by layer, and the order in which layers run).

The reference keeps one flat `Config` for every model and matches names
loosely, falling back to Mistral for anything unknown
(src/loader/mod.rs:36-81, src/model/architecture.rs:59-72,
src/model/models/mod.rs:93-98); here an unknown name is an error that lists
the registered ones.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Optional


class ConfigError(ValueError):
    """A config.json that cannot be used: a missing or ill-typed key, a value
    outside what the architecture allows, or an unknown architecture."""


@dataclass
class ModelConfig:
    """Base of every architecture's configuration."""
    architecture: str = ""
    extra: Dict[str, Any] = field(default_factory=dict)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


@dataclass
class ArchitectureEntry:
    name: str
    config_cls: type
    build_spec: Callable[[ModelConfig], Any]


_ARCHITECTURES: Dict[str, ArchitectureEntry] = {}


def register_architecture(name: str, config_cls: type, build_spec: Callable) -> None:
    """Register `name` (as written in config.json's `architectures`)."""
    _ARCHITECTURES[name] = ArchitectureEntry(name, config_cls, build_spec)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> ArchitectureEntry:
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def architecture_name(d: Dict[str, Any]) -> str:
    archs = d.get("architectures")
    if not isinstance(archs, (list, tuple)) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a non-empty list of names")
    return archs[0]


def config_from_dict(d: Dict[str, Any]) -> ModelConfig:
    entry = get_architecture(architecture_name(d))
    return entry.config_cls.from_dict(d)


def load_config(model_dir: str) -> ModelConfig:
    """Read `<model_dir>/config.json` into the configuration class of the
    architecture it names."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir!r}")
    with open(path, "r") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return config_from_dict(d)


# ---- helpers for config classes -------------------------------------------

def take_int(d, key, default=None, required=False, minimum=None, allow_none=False) -> Optional[int]:
    if key not in d or (d[key] is None and not allow_none and default is not None):
        if required:
            raise ConfigError(f"config.json: missing key {key!r}")
        return default
    v = d[key]
    if v is None:
        if allow_none:
            return None
        if required:
            raise ConfigError(f"config.json: {key!r} must not be null")
        return default
    if isinstance(v, bool) or not isinstance(v, int):
        if isinstance(v, float) and v == int(v):
            v = int(v)
        else:
            raise ConfigError(f"config.json: {key!r} must be an integer, got {v!r}")
    if minimum is not None and v < minimum:
        raise ConfigError(f"config.json: {key!r} must be >= {minimum}, got {v}")
    return v


def take_float(d, key, default=None, required=False, positive=False) -> Optional[float]:
    if key not in d or d[key] is None:
        if required:
            raise ConfigError(f"config.json: missing key {key!r}")
        return default
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {key!r} must be a number, got {v!r}")
    v = float(v)
    if positive and not v > 0.0:
        raise ConfigError(f"config.json: {key!r} must be > 0, got {v}")
    return v


def take_bool(d, key, default=False) -> bool:
    if key not in d or d[key] is None:
        return default
    v = d[key]
    if not isinstance(v, bool):
        raise ConfigError(f"config.json: {key!r} must be true or false, got {v!r}")
    return v
