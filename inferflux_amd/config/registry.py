"""The one registry from an architecture's name to its model.

An architecture is registered as (config class, plan builder): the config class parses
config.json, the plan builder turns the typed config into a ``ModelPlan`` (a list of
layers made of parts, and the order they run in).  Lookup goes by ``model_type`` and then
by ``architectures[0]``, the order the reference uses
(runtime/backends/cuda/inferflux_cuda_executor.cpp:576-583); an unknown name is an error
that lists what is registered (the reference returns nullptr and logs "Unsupported
model_type", runtime/backends/cuda/native/model_forward_factory.cpp:46-60).
"""
from __future__ import annotations

from typing import Any, Callable, Dict, Mapping, Tuple, Type

from .base import ConfigError, ModelConfig, read_config_json

_ARCHITECTURES: Dict[str, Tuple[Type[ModelConfig], Callable]] = {}


def register_architecture(config_cls: Type[ModelConfig], plan_builder: Callable, *extra_names: str) -> None:
    """Register ``config_cls`` under its model_type, its architectures and ``extra_names``."""
    names = [config_cls.model_type, *config_cls.architectures, *extra_names]
    names = [n for n in names if n]
    if not names:
        raise ValueError(f"{config_cls.__name__} names no model_type and no architectures")
    for n in names:
        key = n.lower()
        prev = _ARCHITECTURES.get(key)
        if prev is not None and prev[0] is not config_cls:
            raise ValueError(f"architecture name '{n}' is already registered for {prev[0].__name__}")
        _ARCHITECTURES[key] = (config_cls, plan_builder)


def _ensure_builtin() -> None:
    """The built-in architectures register themselves when their package is imported."""
    from .. import architectures  # noqa: F401


def registered_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def resolve_architecture(d: Mapping[str, Any]) -> Tuple[Type[ModelConfig], Callable]:
    _ensure_builtin()
    candidates = []
    mt = d.get("model_type")
    if isinstance(mt, str) and mt:
        candidates.append(mt)
    archs = d.get("architectures")
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        candidates.append(archs[0])
    if not candidates:
        raise ConfigError("config.json names neither 'model_type' nor 'architectures'")
    for c in candidates:
        hit = _ARCHITECTURES.get(c.lower())
        if hit is not None:
            return hit
    raise ConfigError(
        f"unsupported architecture {candidates!r}; registered: {', '.join(registered_architectures())}")


def config_from_dict(d: Mapping[str, Any]) -> ModelConfig:
    cls, _ = resolve_architecture(d)
    return cls.from_dict(d)


def load_config(folder: str) -> ModelConfig:
    return config_from_dict(read_config_json(folder))


def plan_for(config: ModelConfig):
    """The ModelPlan of a typed config, through the architecture's registered builder."""
    _ensure_builtin()
    hit = _ARCHITECTURES.get(config.model_type.lower())
    if hit is None:
        raise ConfigError(f"architecture '{config.model_type}' is not registered")
    return hit[1](config)
