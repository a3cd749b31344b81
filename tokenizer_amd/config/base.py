"""Typed model configurations read from `config.json`."""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json that cannot describe a model this framework can build."""


_MISSING = dataclasses.MISSING


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's configuration.

    A subclass is a frozen dataclass whose field names are the architecture's
    own config.json keys.  Fields without a default are required keys; unknown
    keys are ignored (the reference ignores them too, qwen-infer/src/model.rs:25).
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ModelConfig":
        values = {}
        missing = []
        for field in dataclasses.fields(cls):
            if field.name in raw and raw[field.name] is not None:
                values[field.name] = _coerce(field, raw[field.name])
            elif field.default is _MISSING and field.default_factory is _MISSING:
                missing.append(field.name)
        if missing:
            raise ConfigError(f"config.json for {cls.architecture or cls.__name__} lacks required keys: "
                              + ", ".join(missing))
        cfg = cls(**values)
        cfg.validate()
        return cfg

    def validate(self) -> None:  # pragma: no cover - overridden
        pass

    def to_dict(self) -> dict[str, Any]:
        out = {"architectures": [self.architecture]}
        for field in dataclasses.fields(self):
            value = getattr(self, field.name)
            if value is not None:
                out[field.name] = value
        return out

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as fh:
            json.dump(self.to_dict(), fh, indent=1)


def _coerce(field: dataclasses.Field, value: Any) -> Any:
    kind = field.type if isinstance(field.type, str) else getattr(field.type, "__name__", str(field.type))
    kind = kind.replace(" ", "").replace("|None", "")
    try:
        if kind == "int":
            if isinstance(value, bool) or (isinstance(value, float) and value != int(value)):
                raise ValueError
            return int(value)
        if kind == "float":
            if isinstance(value, bool):
                raise ValueError
            return float(value)
        if kind == "bool":
            if not isinstance(value, bool):
                raise ValueError
            return value
        if kind == "str":
            if not isinstance(value, str):
                raise ValueError
            return value
    except (TypeError, ValueError):
        raise ConfigError(f"config.json key {field.name!r} should be {kind}, found {value!r}") from None
    return value


def read_config_json(folder_or_file: str) -> dict[str, Any]:
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as fh:
            raw = json.load(fh)
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    except json.JSONDecodeError as err:
        raise ConfigError(f"{path} is not valid JSON: {err}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw
