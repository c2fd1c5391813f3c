"""One registry from an architecture's name (``architectures[0]`` of config.json) to its
typed configuration class.  A configuration class has ``from_dict(raw) -> config``,
``config.to_spec() -> ModelSpec`` and, for the random-weights mode,
``config.random_tensor_plan()`` and ``config.to_dict()``.

The reference has no registry: it switches on flags inside one forward function
(``crates/mach-model/src/batched.rs:3201, 3405, 4055``).
"""
from __future__ import annotations

import json
import os
from typing import Dict

from .specs import ConfigError

_ARCHITECTURES: Dict[str, type] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: type, model_type: str | None = None) -> None:
    _ARCHITECTURES[name] = config_cls
    if model_type:
        _MODEL_TYPES[model_type] = name


def architectures() -> list:
    return sorted(_ARCHITECTURES)


def architecture_of(raw: dict) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        name = archs[0]
    elif isinstance(raw.get("model_type"), str) and raw["model_type"] in _MODEL_TYPES:
        name = _MODEL_TYPES[raw["model_type"]]
    else:
        raise ConfigError("config.json: no 'architectures' list and no known 'model_type'; "
                          f"supported architectures: {architectures()}")
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config.json: architecture {name!r} is not supported; supported: {architectures()}")
    return name


def config_from_dict(raw: dict):
    return _ARCHITECTURES[architecture_of(raw)].from_dict(raw)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json") if os.path.isdir(model_dir) else model_dir
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return config_from_dict(raw)
