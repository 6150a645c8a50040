"""One registry from the architecture name in config.json to its model.

An architecture is a function from the config.json dictionary to a typed
configuration object that has ``to_model_spec()`` and ``to_dict()``.
"""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict

from .qwen3 import ARCHITECTURE as _QWEN3, ConfigError, Qwen3Config

_ARCHITECTURES: Dict[str, Callable[[Dict[str, Any]], Any]] = {}


def register_architecture(name: str, from_dict: Callable[[Dict[str, Any]], Any]) -> None:
    _ARCHITECTURES[name] = from_dict


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any]):
    archs = d.get("architectures")
    if not archs:
        raise ConfigError("config.json has no 'architectures' entry; known: "
                          + ", ".join(known_architectures()))
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; known: "
                          + ", ".join(known_architectures()))
    return _ARCHITECTURES[name](d)


def config_from_folder(folder: str):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder}")
    with open(path) as f:
        return config_from_dict(json.load(f))


register_architecture(_QWEN3, Qwen3Config.from_dict)
