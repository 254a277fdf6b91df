"""One registry: architecture name (config.json `architectures[0]`) -> config class.

A config class has `from_dict(dict) -> config` and the config has
`to_dict()`, `validate()` and `model_spec() -> ModelSpec`.  An unknown name is an
error that lists the known ones, never a fallback (reference:
`ParseArchitecture`, `src/model/config.cc:40-54`; the factory switch
`src/engine/model_runner_factory.cc:237-259`).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Type

_ARCHITECTURES: Dict[str, Type] = {}


class ConfigError(ValueError):
    """config.json is missing a key, has a wrong type or an impossible value."""


def register_architecture(name: str, config_cls: Type) -> None:
    _ARCHITECTURES[name] = config_cls


def known_architectures():
    return sorted(_ARCHITECTURES)


def config_class_for(name: str) -> Type:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture {name!r}; known: {', '.join(known_architectures()) or '(none)'}"
        ) from None


def config_from_dict(raw: Dict[str, Any]):
    archs = raw.get("architectures")
    if not isinstance(archs, list) or len(archs) != 1 or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a list with exactly one name")
    cfg = config_class_for(archs[0]).from_dict(raw)
    cfg.validate()
    return cfg


def config_from_json(text: str):
    try:
        raw = json.loads(text)
    except json.JSONDecodeError as e:
        raise ConfigError(f"config.json is not valid JSON: {e}") from None
    if not isinstance(raw, dict):
        raise ConfigError("config.json must hold a JSON object")
    return config_from_dict(raw)


def config_from_directory(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file")
    with open(path, "r", encoding="utf-8") as f:
        return config_from_json(f.read())
