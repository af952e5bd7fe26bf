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
    raw = json.loads(path.read_text())
    # a checkpoint's generation_config.json may name more stop tokens than config.json (a chat model's end-of-turn
    # token beside the end-of-text one); generation stops at any of them
    extra = Path(model_dir) / "generation_config.json"
    if extra.is_file():
        more = json.loads(extra.read_text()).get("eos_token_id")
        if more is not None:
            ids = []
            for group in (raw.get("eos_token_id"), more):
                for t in ([] if group is None else group if isinstance(group, (list, tuple)) else [group]):
                    if int(t) not in ids:
                        ids.append(int(t))
            raw = dict(raw, eos_token_id=ids)
    return config_from_dict(raw)


# ---- named sizes -------------------------------------------------------------------------------------
# config.json files kept as data beside this module: the sizes that measurements and examples name
# (the reference names models by package file; its benchmark protocol is examples/bench.cpp:564-590).
PRESET_DIR = Path(__file__).resolve().parent / "presets"


def preset_names() -> list[str]:
    return sorted(p.stem for p in PRESET_DIR.glob("*.json"))


def preset_dict(name: str) -> dict:
    """The config.json of a named size, as a dict."""
    path = PRESET_DIR / f"{name}.json"
    if not path.is_file():
        raise ConfigError(f"unknown size {name!r}; known: {', '.join(preset_names())}")
    return json.loads(path.read_text())


def config_source(name_or_path) -> dict:
    """A config.json given as a path to the file (or to its folder), or as a named size."""
    path = Path(name_or_path)
    if path.is_dir():
        path = path / "config.json"
    if path.is_file():
        return json.loads(path.read_text())
    return preset_dict(str(name_or_path))
