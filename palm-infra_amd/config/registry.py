"""One registry from an architecture's name to its configuration class (and through it, its model).

The reference keeps a table from ``model_type`` to a converter function and prints the supported
list for an unknown type (models/converter.py:24-46).  Here the key is ``architectures[0]`` of
config.json, with ``model_type`` as a second way in.
"""
from __future__ import annotations

import json
from pathlib import Path


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value the architecture cannot run with."""


_BY_ARCHITECTURE: dict[str, type] = {}
_BY_MODEL_TYPE: dict[str, type] = {}


def register_architecture(name: str, model_type: str | None = None):
    def deco(cls):
        if name in _BY_ARCHITECTURE and _BY_ARCHITECTURE[name] is not cls:
            raise ValueError(f"architecture {name!r} is already registered")
        _BY_ARCHITECTURE[name] = cls
        if model_type is not None:
            _BY_MODEL_TYPE[model_type] = cls
        cls.architecture = name
        cls.model_type = model_type
        return cls
    return deco


def registered_architectures() -> list[str]:
    return sorted(_BY_ARCHITECTURE)


def config_class_for(raw: dict) -> type:
    archs = raw.get("architectures") or []
    for a in archs:
        if a in _BY_ARCHITECTURE:
            return _BY_ARCHITECTURE[a]
    mt = raw.get("model_type")
    if not archs and mt in _BY_MODEL_TYPE:
        return _BY_MODEL_TYPE[mt]
    named = archs[0] if archs else mt
    raise ConfigError(f"unknown architecture {named!r}; registered: {', '.join(registered_architectures())}")


def config_from_dict(raw: dict):
    return config_class_for(raw).from_dict(raw)


def config_from_dir(model_dir):
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json in {model_dir}")
    return config_from_dict(json.loads(path.read_text()))
