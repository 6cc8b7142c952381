"""Typed model configuration: the base class every architecture's config derives from.

A configuration is read from the keys of the architecture's own ``config.json`` and
nothing else; every size and constant the model uses comes from it.  The reference
keeps an untyped struct that is silently zero when ``config.json`` is missing or a
key is absent (runtime/backends/cuda/inferflux_cuda_executor.cpp:358-361, 543-598);
here a missing required key, a wrong type or an inconsistent combination is an error
that names the key.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar, Dict, Mapping, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a runnable model."""


_MISSING = object()


def read_key(d: Mapping[str, Any], key: str, kind, default: Any = _MISSING):
    """Return ``d[key]`` converted to ``kind`` (int, float, bool, str).

    Raises ConfigError when the key is absent and has no default, or when the value
    has the wrong JSON type (a bool is not accepted for a number, nor the reverse).
    """
    if key not in d or d[key] is None:
        if default is _MISSING:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    v = d[key]
    if kind is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"config.json: '{key}' must be true/false, got {v!r}")
        return v
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                return int(v)
            raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
        return v
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: '{key}' must be a number, got {v!r}")
        return float(v)
    if kind is str:
        if not isinstance(v, str):
            raise ConfigError(f"config.json: '{key}' must be a string, got {v!r}")
        return v
    raise TypeError(kind)


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    """Base of all architecture configurations.

    Subclasses are frozen dataclasses whose fields carry the names of the config.json
    keys.  ``model_type`` and ``architectures`` are the names under which the
    architecture registry finds the subclass.
    """

    model_type: ClassVar[str] = ""
    architectures: ClassVar[Tuple[str, ...]] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        """The config.json content that ``from_dict`` reads back to an equal object."""
        out: Dict[str, Any] = {
            "model_type": self.model_type,
            "architectures": list(self.architectures[:1]),
        }
        for f in dataclasses.fields(self):
            out[f.name] = getattr(self, f.name)
        return out

    def validate(self) -> None:
        raise NotImplementedError

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)
            f.write("\n")


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder}: no config.json (a model folder holds config.json and model.safetensors)")
    try:
        with open(path) as f:
            d = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d
