"""Typed model configurations read from an architecture's own config.json keys."""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, fields
from typing import Any, ClassVar, Mapping


class ConfigError(ValueError):
    """A config.json that names something the engine cannot run, or lacks a required key."""


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    try:
        with open(path) as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"No config.json in model folder {folder!r}.") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}.") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} must hold a JSON object.")
    return raw


def positive_int(raw: Mapping[str, Any], key: str) -> int:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"Invalid model config: {key} must be a positive integer, got {value!r}.")
    return value


def positive_float(raw: Mapping[str, Any], key: str) -> float:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) or value <= 0:
        raise ConfigError(f"Invalid model config: {key} must be a positive finite number, got {value!r}.")
    return float(value)


def token_id_list(value: Any, vocab_size: int, key: str) -> tuple[int, ...]:
    ids = value if isinstance(value, list) else [value]
    if not ids or any(isinstance(i, bool) or not isinstance(i, int) or i < 0 or i >= vocab_size for i in ids):
        raise ConfigError(f"Invalid {key}: every id must be an integer in [0, {vocab_size}).")
    return tuple(dict.fromkeys(ids))


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's configuration.

    A subclass names its architecture, parses its own config.json keys in
    `from_dict` (no defaults for sizes or constants) and writes them back in
    `to_dict`, so that a configuration can be saved as a model folder.
    """

    architecture: ClassVar[str] = ""
    model_types: ClassVar[tuple[str, ...]] = ()

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict:
        raise NotImplementedError

    def replace(self, **changes) -> "ModelConfig":
        values = {f.name: getattr(self, f.name) for f in fields(self)}
        values.update(changes)
        return type(self).from_dict(type(self)(**values).to_dict())
