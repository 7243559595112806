"""One registry from an architecture's name to its typed configuration.

``config.json`` names its architecture in ``architectures[0]`` (and ``model_type``);
the registered configuration class reads that file's keys and lowers them to a
:class:`ModelSpec`, from which the generic model is built. The reference selects its
plan builder with a chain of string compares and refuses unknown names
(native/src/v2_runtime.cpp:19898-19915,20050-20057).
"""

from __future__ import annotations

import os
from typing import Any, Dict, Mapping, Type

from . import json_reader
from .spec import ConfigError

_ARCHITECTURES: Dict[str, Type] = {}


def register_architecture(name: str, config_class: Type, *, replace: bool = False) -> None:
    """``config_class`` must offer ``from_dict(mapping)`` and ``model_spec()``."""
    for method in ("from_dict", "model_spec"):
        if not hasattr(config_class, method):
            raise TypeError(f"{config_class.__name__} lacks {method}()")
    if name in _ARCHITECTURES and not replace and _ARCHITECTURES[name] is not config_class:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = config_class


def registered_architectures() -> tuple:
    return tuple(sorted(_ARCHITECTURES))


def architecture_name(data: Mapping[str, Any]) -> str:
    names = data.get("architectures")
    if isinstance(names, list) and names and isinstance(names[0], str):
        return names[0]
    model_type = data.get("model_type")
    if isinstance(model_type, str):
        return model_type
    raise ConfigError("config.json is missing 'architectures' (and 'model_type')")


def config_from_dict(data: Mapping[str, Any]):
    if not isinstance(data, Mapping):
        raise ConfigError("config.json must hold a JSON object")
    name = architecture_name(data)
    config_class = _ARCHITECTURES.get(name)
    if config_class is None and isinstance(data.get("model_type"), str):
        config_class = _ARCHITECTURES.get(data["model_type"])
    if config_class is None:
        raise ConfigError(
            f"unknown architecture '{name}'; registered: {', '.join(registered_architectures()) or 'none'}")
    return config_class.from_dict(data)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir}: no config.json")
    try:
        data = json_reader.parse_file(path)
    except json_reader.JsonError as error:
        raise ConfigError(f"{path}: {error}") from None
    return config_from_dict(data)
