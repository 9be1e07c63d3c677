"""The one registry from an architecture's name to its model.

An entry holds the configuration class that reads the architecture's config.json
and the function that turns that configuration into a ``ModelSpec`` (the list of
layers, their parts and the order they run in).  The reference dispatches on
``architectures[0]`` and falls back to ``model_type`` (src/models/config.rs:139-145).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Type

from ..errors import UnsupportedError
from .base import ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Type[ModelConfig]
    build_spec: Callable            # (config) -> parts.spec.ModelSpec


_BY_NAME: dict[str, Architecture] = {}
_ALIASES: dict[str, str] = {}


def register_architecture(name: str, config_class, build_spec, model_types=()) -> Architecture:
    """Add (or replace) an architecture.  ``model_types`` are config.json
    ``model_type`` values that select it when ``architectures`` is absent."""
    arch = Architecture(name, config_class, build_spec)
    _BY_NAME[name] = arch
    for alias in model_types:
        _ALIASES[alias] = name
    return arch


def known_architectures() -> list[str]:
    return sorted(_BY_NAME)


def resolve_architecture(raw: dict) -> Architecture:
    """The registry entry a config.json selects, by ``architectures[0]`` and else by
    ``model_type``; an unknown name is an error that lists the known ones."""
    archs = raw.get("architectures") or []
    name = archs[0] if archs else None
    if name is None:
        name = _ALIASES.get(raw.get("model_type"))
    if name not in _BY_NAME:
        asked = archs[0] if archs else raw.get("model_type")
        raise UnsupportedError(f"architecture {asked!r} is not registered; known: {', '.join(known_architectures())}")
    return _BY_NAME[name]


def config_from_dict(raw: dict):
    """(architecture entry, typed configuration) for a parsed config.json."""
    arch = resolve_architecture(raw)
    return arch, arch.config_class.from_dict(raw)


def load_config(model_dir: str):
    return config_from_dict(read_config_json(model_dir))
