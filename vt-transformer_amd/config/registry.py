"""One registry from the architecture's name (config.json `architectures[0]`)
to its configuration class.

The reference has no such map: each model is a folder with its own program
(v1/models/*/inference_fp16.dag); its only name->factory table is the word
table of the interpreter (v1/tensortype/dag.hpp:389-394).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Type

from .base import ConfigError, ModelConfig

_ARCHITECTURES: Dict[str, Type[ModelConfig]] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig]) -> None:
    """Make `name` known.  `config_cls.from_dict` reads that architecture's
    config.json, `to_spec` says which parts its layers are made of."""
    _ARCHITECTURES[name] = config_cls


def architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any]) -> ModelConfig:
    archs = d.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: key 'architectures' must be a list holding the architecture's name")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config.json: architecture '{name}' is not registered (known: {', '.join(architectures())})")
    return _ARCHITECTURES[name].from_dict(d)


def load_config(folder: str) -> ModelConfig:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder}: no config.json")
    with open(path) as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return config_from_dict(d)
