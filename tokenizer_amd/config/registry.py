"""One registry from an architecture's name to its configuration and model.

The name is `config.json:architectures[0]`.  An architecture registers a
configuration class and a function that turns a configuration into a
`ModelSpec` (the list of layers, their parts and the order they run in).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable

from .base import ConfigError, ModelConfig, read_config_json


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable[[Any], Any]


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, build_spec: Callable[[Any], Any],
                          replace: bool = False) -> Architecture:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    config_class.architecture = name
    arch = Architecture(name, config_class, build_spec)
    _ARCHITECTURES[name] = arch
    return arch


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"unknown architecture {name!r}; registered: "
                          + ", ".join(registered_architectures())) from None


def architecture_name(raw: dict[str, Any]) -> str:
    names = raw.get("architectures")
    if not isinstance(names, list) or not names or not isinstance(names[0], str):
        raise ConfigError("config.json has no `architectures` list naming the model class; registered: "
                          + ", ".join(registered_architectures()))
    return names[0]


def load_config(folder_or_file: str) -> ModelConfig:
    """Read config.json and build the typed configuration its architecture registered."""
    raw = read_config_json(folder_or_file)
    arch = get_architecture(architecture_name(raw))
    return arch.config_class.from_dict(raw)
