"""Typed configuration: what every architecture's configuration has in common.

A configuration class reads the keys of its architecture's own ``config.json`` and
nothing else decides a size or a constant of the model.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields
from typing import Any, ClassVar

import numpy as np

from ..errors import ConfigError

_MISSING = object()


def f32(value: Any, key: str) -> float:
    """A number as the nearest 32-bit float: the reference parses ``rms_norm_eps`` and
    ``rope_theta`` as f32 (src/models/config.rs:31-34), and the rotation's
    frequencies are computed from that 32-bit theta."""
    try:
        return float(np.float32(value))
    except (TypeError, ValueError):
        raise ConfigError(f"config key {key!r}: expected a number, got {value!r}") from None


def whole(value: Any, key: str, minimum: int = 0) -> int:
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config key {key!r}: expected an integer, got {value!r}")
    if value < minimum:
        raise ConfigError(f"config key {key!r}: {value} is below {minimum}")
    return value


@dataclass(frozen=True)
class ModelConfig:
    """Base of the typed configurations.  Subclasses list their keys as dataclass
    fields, name required ones in ``REQUIRED`` and implement ``validate``."""

    ARCHITECTURE: ClassVar[str] = ""
    MODEL_TYPE: ClassVar[str] = ""
    REQUIRED: ClassVar[tuple[str, ...]] = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "ModelConfig":
        raise NotImplementedError

    def validate(self) -> None:
        raise NotImplementedError

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {"architectures": [self.ARCHITECTURE], "model_type": self.MODEL_TYPE}
        for f in fields(self):
            v = getattr(self, f.name)
            if v is not None:
                out[f.name] = v
        return out

    @classmethod
    def require(cls, raw: dict) -> None:
        missing = [k for k in cls.REQUIRED if k not in raw]
        if missing:
            raise ConfigError(f"config.json for {cls.ARCHITECTURE} lacks {', '.join(missing)}")


def read_config_json(model_dir: str) -> dict:
    """The parsed config.json of a model folder; errors name the path
    (src/error.rs:6-18 carries the path in its Io and Json variants)."""
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except OSError as e:
        raise ConfigError(f"cannot read {path}: {e.strerror or e}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return raw
