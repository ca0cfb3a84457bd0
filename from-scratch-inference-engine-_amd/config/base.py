"""What every typed configuration shares: errors, the JSON file and field helpers."""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Mapping


class ConfigError(ValueError):
    """config.json is missing a key, holds a value the engine cannot run, or names an
    architecture that is not registered."""


@dataclass(frozen=True)
class ModelConfig:
    """Base of the typed configurations.  A subclass holds every size and constant of one
    architecture, read from that architecture's own config.json keys; nothing else in the
    engine hard-codes them."""

    architecture: str

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ModelConfig":  # pragma: no cover - abstract
        raise NotImplementedError

    def to_dict(self) -> dict:  # pragma: no cover - abstract
        """config.json content that ``from_dict`` reads back to an equal configuration."""
        raise NotImplementedError


def read_config_json(model_dir) -> dict:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"no config.json in {model_dir}")
    try:
        raw = json.loads(path.read_text(encoding="utf-8"))
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: invalid JSON: {e}") from e
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def required_int(raw: Mapping[str, Any], key: str, minimum: int = 1) -> int:
    if key not in raw:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    return checked_int(raw[key], key, minimum)


def checked_int(value: Any, key: str, minimum: int = 1) -> int:
    if isinstance(value, bool) or not isinstance(value, (int, float)) or int(value) != value:
        raise ConfigError(f"config.json: '{key}' must be an integer, found {value!r}")
    value = int(value)
    if value < minimum:
        raise ConfigError(f"config.json: '{key}' must be >= {minimum}, found {value}")
    return value


def checked_float(value: Any, key: str, positive: bool = True) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json: '{key}' must be a number, found {value!r}")
    value = float(value)
    if positive and not value > 0.0:
        raise ConfigError(f"config.json: '{key}' must be > 0, found {value}")
    return value
