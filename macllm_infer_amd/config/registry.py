"""One registry from an architecture's name to its configuration class.

``config.json`` names its architecture in ``architectures[0]`` (or ``model_type``);
the class registered under that name reads the rest of the file and lowers it to a
``ModelSpec``.  The reference resolves a file the same way: architecture string ->
spec builder -> adapter (src/gguf_model.rs:315-354, :391-444), and an unknown name is
an error that lists the supported ones (src/models/mod.rs:698-714).

A configuration class must offer ``from_dict(raw) -> config`` (validated),
``to_model_spec() -> ModelSpec``, ``to_dict()`` and ``architecture_names``.
"""
from __future__ import annotations

import json
import os
from typing import Dict

from .spec import ConfigError

_ARCHITECTURES: Dict[str, type] = {}


def register_architecture(config_class: type) -> type:
    """Register ``config_class`` under each of its ``architecture_names`` (usable as a decorator)."""
    for name in config_class.architecture_names:
        _ARCHITECTURES[name] = config_class
    return config_class


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(raw: dict):
    names = []
    architectures = raw.get("architectures")
    if isinstance(architectures, list) and architectures:
        names.append(architectures[0])
    if isinstance(raw.get("model_type"), str):
        names.append(raw["model_type"])
    if not names:
        raise ConfigError("config.json names no architecture ('architectures' or 'model_type'); "
                          f"registered: {registered_architectures()}")
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name].from_dict(raw)
    raise ConfigError(f"unknown architecture {names[0]!r}; registered: {registered_architectures()}")


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path} does not exist")
    with open(path) as handle:
        try:
            raw = json.load(handle)
        except json.JSONDecodeError as error:
            raise ConfigError(f"{path} is not valid JSON: {error}") from error
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return config_from_dict(raw)
