"""The one registry from an architecture's name to its configuration class and model builder.

The reference maps a file's architecture string to a model class and rejects
unknown names with the name in the error (crates/leone/src/model.rs:23-31,
crates/leone-gguf/src/support.rs:39-56).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping

from ..config.base import UnsupportedArchitecture, architecture_name, read_config_json
from ..parts.model import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Mapping[str, Any]], Any]
    model_spec: Callable[[Any], ModelSpec]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, model_spec) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_from_dict, model_spec)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def lookup(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnsupportedArchitecture(name, known_architectures()) from None


def config_from_dict(raw: Mapping[str, Any]):
    """The typed configuration for a config.json mapping, chosen by its architecture name."""
    return lookup(architecture_name(raw)).config_from_dict(raw)


def config_from_dir(model_dir: str):
    return config_from_dict(read_config_json(model_dir))


def model_spec_for(config) -> ModelSpec:
    return lookup(config.architecture).model_spec(config)
