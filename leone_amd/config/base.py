"""Typed model configuration: shared errors and field readers.

An architecture's configuration class reads the keys of that architecture's own
``config.json`` and nothing else; every size and constant a part needs reaches
it through such a class.  The checks follow the reference's metadata validation
(crates/leone-gguf/src/model.rs:135-172: nonzero sizes, grouped-query
divisibility, finite positive floats) and its typed errors
(crates/leone-gguf/src/model.rs:59-79).
"""
from __future__ import annotations

import json
import math
import os
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json that cannot be used; ``field`` names the offending key."""

    def __init__(self, field: str, message: str):
        super().__init__(f"config.json: {field}: {message}")
        self.field = field


class UnsupportedArchitecture(ConfigError):
    def __init__(self, name: Any, known: list[str]):
        super().__init__(
            "architectures",
            f"unsupported architecture {name!r}; registered: {', '.join(sorted(known)) or '(none)'}",
        )
        self.name = name
        self.known = list(known)


_MISSING = object()


class FieldReader:
    """Reads typed fields from a config.json mapping and records what was used."""

    def __init__(self, raw: Mapping[str, Any]):
        self.raw = raw
        self.used: set[str] = set()

    def has(self, key: str) -> bool:
        return key in self.raw and self.raw[key] is not None

    def _get(self, key: str, default: Any) -> Any:
        self.used.add(key)
        value = self.raw.get(key, _MISSING)
        if value is _MISSING or value is None:
            if default is _MISSING:
                raise ConfigError(key, "required key is missing")
            return default
        return value

    def positive_int(self, key: str, default: Any = _MISSING) -> int:
        value = self._get(key, default)
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(key, f"expected an integer, found {value!r}")
        if value <= 0:
            raise ConfigError(key, f"must be positive, found {value}")
        return value

    def positive_float(self, key: str, default: Any = _MISSING) -> float:
        value = self._get(key, default)
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(key, f"expected a number, found {value!r}")
        value = float(value)
        if not math.isfinite(value) or value <= 0.0:
            raise ConfigError(key, f"must be finite and positive, found {value}")
        return value

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        value = self._get(key, default)
        if not isinstance(value, bool):
            raise ConfigError(key, f"expected true or false, found {value!r}")
        return value

    def optional(self, key: str) -> Any:
        self.used.add(key)
        return self.raw.get(key)

    def string(self, key: str, default: Any = _MISSING) -> str:
        value = self._get(key, default)
        if not isinstance(value, str):
            raise ConfigError(key, f"expected a string, found {value!r}")
        return value


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as handle:
            raw = json.load(handle)
    except FileNotFoundError:
        raise ConfigError("config.json", f"no such file: {path}") from None
    except json.JSONDecodeError as error:
        raise ConfigError("config.json", f"not valid JSON: {error}") from None
    if not isinstance(raw, dict):
        raise ConfigError("config.json", "top level must be an object")
    return raw


def architecture_name(raw: Mapping[str, Any]) -> str:
    """The registry key of a config.json: ``architectures[0]``."""
    names = raw.get("architectures")
    if not isinstance(names, list) or len(names) != 1 or not isinstance(names[0], str):
        raise ConfigError("architectures", f"expected a list with one name, found {names!r}")
    return names[0]
