"""The one registry from an architecture's name to its configuration class and its model plan."""
from __future__ import annotations

from typing import Callable, Mapping

from .config.base import ConfigError, ModelConfig, read_config_json

_ARCHITECTURES: dict[str, tuple[type, Callable]] = {}
_MODEL_TYPES: dict[str, str] = {}


def register_architecture(name: str, config_cls: type, builder: Callable, model_types=()) -> None:
    """`builder(config) -> ModelPlan`.  `model_types` are config.json `model_type` values that select
    this architecture when `architectures` is absent."""
    _ARCHITECTURES[name] = (config_cls, builder)
    for model_type in model_types or getattr(config_cls, "model_types", ()):
        _MODEL_TYPES[model_type] = name


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(raw: Mapping) -> str:
    names = raw.get("architectures")
    if isinstance(names, list) and names:
        for name in names:
            if name in _ARCHITECTURES:
                return name
        raise ConfigError(f"Unknown architecture {names!r}; registered: {registered_architectures()}.")
    model_type = raw.get("model_type")
    if model_type in _MODEL_TYPES:
        return _MODEL_TYPES[model_type]
    raise ConfigError(f"config.json names no known architecture (architectures={names!r}, "
                      f"model_type={model_type!r}); registered: {registered_architectures()}.")


def config_from_dict(raw: Mapping) -> ModelConfig:
    config_cls, _ = _ARCHITECTURES[resolve_architecture(raw)]
    return config_cls.from_dict(raw)


def load_config(folder: str) -> ModelConfig:
    return config_from_dict(read_config_json(folder))


def build_model_plan(config: ModelConfig):
    try:
        _, builder = _ARCHITECTURES[config.architecture]
    except KeyError:
        raise ConfigError(f"Unknown architecture {config.architecture!r}; registered: "
                          f"{registered_architectures()}.") from None
    return builder(config)


def _register_builtin():
    from .config.qwen2 import Qwen2Config
    from .models.qwen2 import build_qwen2
    register_architecture(Qwen2Config.architecture, Qwen2Config, build_qwen2)


_register_builtin()
