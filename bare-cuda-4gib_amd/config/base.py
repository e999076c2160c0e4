"""Typed configuration read from an architecture's own config.json keys."""
from __future__ import annotations

import dataclasses
import json
import math
import os
from typing import Any, Dict

from ..errors import ConfigError

_MISSING = dataclasses.MISSING


def field_from_json(key: str, default: Any = _MISSING, doc: str = ""):
    """A dataclass field filled from ``config.json[key]``.

    Without a default the key is required.
    """
    meta = {"json_key": key, "doc": doc}
    if default is _MISSING:
        return dataclasses.field(metadata=meta)
    return dataclasses.field(default=default, metadata=meta)


def _coerce(name: str, key: str, value: Any, typ: Any) -> Any:
    if typ in ("int", int):
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                return int(value)
            raise ConfigError(f"config.json: '{key}' must be an integer, got {value!r}")
        return value
    if typ in ("float", float):
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"config.json: '{key}' must be a number, got {value!r}")
        value = float(value)
        if not math.isfinite(value):
            raise ConfigError(f"config.json: '{key}' must be finite, got {value!r}")
        return value
    if typ in ("bool", bool):
        if not isinstance(value, bool):
            raise ConfigError(f"config.json: '{key}' must be true or false, got {value!r}")
        return value
    if typ in ("str", str):
        if not isinstance(value, str):
            raise ConfigError(f"config.json: '{key}' must be a string, got {value!r}")
        return value
    return value  # Optional[...] and other loose types: validate() checks them


@dataclasses.dataclass
class ModelConfig:
    """Base of every architecture's configuration.

    A subclass is a dataclass whose fields are declared with
    :func:`field_from_json`; :meth:`from_dict` fills them from the parsed
    config.json, applies defaults for absent optional keys, derives what the
    architecture derives, and validates.  ``raw`` keeps the parsed file.
    """

    def derive(self, raw: Dict[str, Any]) -> None:
        """Fill fields whose default depends on other fields."""

    def validate(self) -> None:
        """Raise ConfigError for values the architecture cannot express."""

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        if not isinstance(raw, dict):
            raise ConfigError("config.json must hold a JSON object")
        values = {}
        for f in dataclasses.fields(cls):
            key = f.metadata.get("json_key")
            if key is None:
                continue
            if key in raw and raw[key] is not None:
                values[f.name] = _coerce(f.name, key, raw[key], f.type)
            elif f.default is _MISSING and f.default_factory is _MISSING:
                raise ConfigError(f"config.json: required key '{key}' is missing")
        cfg = cls(**values)
        cfg.derive(raw)
        cfg.validate()
        return cfg

    @classmethod
    def from_json_file(cls, path: str) -> "ModelConfig":
        return cls.from_dict(read_config_json(path))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json keys this configuration was (or would be) read from."""
        out = {}
        for f in dataclasses.fields(self):
            key = f.metadata.get("json_key")
            if key is not None:
                out[key] = getattr(self, f.name)
        return out


def read_config_json(path: str) -> Dict[str, Any]:
    """Parse ``path`` (a config.json, or a model folder that holds one)."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as fh:
            return json.load(fh)
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from None
