"""One registry from an architecture's name to its configuration class.

The reference maps `general.architecture` to an enum variant and falls back to
Llama silently for an unknown string (llama3.rs:147-185); here an unknown name
is an error that lists what is registered.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Mapping

from .plan import ConfigError

_ARCHITECTURES: Dict[str, type] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: type, model_type: str = None) -> None:
    """Register a configuration class under config.json's `architectures[0]` name.

    The class needs `from_dict(mapping)`, `to_dict()` and `plan() -> ModelPlan`.
    """
    for attr in ("from_dict", "to_dict", "plan"):
        if not hasattr(config_cls, attr):
            raise TypeError(f"configuration class for '{name}' lacks {attr}()")
    _ARCHITECTURES[name] = config_cls
    if model_type:
        _MODEL_TYPES[model_type] = name


def registered_architectures():
    return sorted(_ARCHITECTURES)


def architecture_name(d: Mapping[str, Any]) -> str:
    archs = d.get("architectures")
    if isinstance(archs, (list, tuple)) and archs and isinstance(archs[0], str):
        name = archs[0]
    elif isinstance(d.get("model_type"), str) and d["model_type"] in _MODEL_TYPES:
        name = _MODEL_TYPES[d["model_type"]]
    else:
        raise ConfigError("config.json: neither 'architectures' nor a known 'model_type' names the "
                          f"architecture; registered: {registered_architectures()}")
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config.json: unknown architecture '{name}'; "
                          f"registered: {registered_architectures()}")
    return name


def config_from_dict(d: Mapping[str, Any]):
    if not isinstance(d, Mapping):
        raise ConfigError("config.json: the top level must be an object")
    return _ARCHITECTURES[architecture_name(d)].from_dict(d)


def load_config(folder_or_file: str):
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    return config_from_dict(d)
