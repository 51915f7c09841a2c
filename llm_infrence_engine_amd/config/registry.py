"""One registry from an architecture's name to its typed configuration (and through it, its model).

``config.json`` names the architecture in ``architectures[0]`` (``model_type`` is the fallback).
The reference has no registry: its loader builds the one model it knows
(src/miniserve/loader.py:38-39) and never reads ``architectures``.
"""
from __future__ import annotations

import json
import sys
from pathlib import Path
from typing import Dict, Type

from .spec import ModelSpec


class ConfigError(ValueError):
    """config.json is missing a key, holds a value the engine cannot run, or names no known architecture."""


_ARCHITECTURES: Dict[str, type] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: type, model_type: str | None = None) -> None:
    """``config_cls`` must offer ``from_dict(dict) -> config``, ``to_dict()`` and ``to_spec() -> ModelSpec``."""
    for attr in ("from_dict", "to_dict", "to_spec"):
        if not hasattr(config_cls, attr):
            raise TypeError(f"{config_cls.__name__} lacks {attr}()")
    _ARCHITECTURES[name] = config_cls
    if model_type:
        _MODEL_TYPES[model_type] = name


def known_architectures() -> list:
    return sorted(_ARCHITECTURES)


def config_class(name: str) -> type:
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; known: {', '.join(known_architectures())}")
    return _ARCHITECTURES[name]


def config_from_dict(d: dict):
    archs = d.get("architectures")
    if archs:
        name = archs[0]
    elif d.get("model_type") in _MODEL_TYPES:
        name = _MODEL_TYPES[d["model_type"]]
    elif len(_ARCHITECTURES) == 1:
        name = next(iter(_ARCHITECTURES))
        print(f"config.json names no architecture; taking the only one known, {name}", file=sys.stderr)
    else:
        raise ConfigError("config.json has neither 'architectures' nor a known 'model_type'; "
                          f"known architectures: {', '.join(known_architectures())}")
    return config_class(name).from_dict(d)


def load_config(model_dir):
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path} not found")
    return config_from_dict(json.loads(path.read_text()))


def build_spec(config) -> ModelSpec:
    return config.to_spec()


def require(d: dict, key: str, kind=None):
    """A required key of config.json, with the key's name in the error."""
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json lacks the required key {key!r}")
    v = d[key]
    if kind is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"config.json: {key!r} must be an integer, got {v!r}")
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: {key!r} must be a number, got {v!r}")
        v = float(v)
    return v
