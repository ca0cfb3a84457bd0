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

    @property
    def max_positions(self) -> int:
        """The most positions a request may reach (0: no limit), from whichever key the
        architecture's config.json keeps it under."""
        return 0

    @property
    def end_token(self) -> int:
        """The end-of-sequence token id of config.json, -1 if it names none."""
        return -1

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


def end_token_of(raw: Mapping[str, Any]) -> int:
    """``eos_token_id`` of a config.json or generation_config.json: an id, the first of a list of
    ids, or -1 where there is none."""
    eos = raw.get("eos_token_id")
    if isinstance(eos, (list, tuple)):
        eos = eos[0] if eos else None
    if eos is None:
        return -1
    return checked_int(eos, "eos_token_id", -1)


def generation_end_token(model_dir) -> int:
    """The end token that the folder's generation_config.json names (it goes before config.json's,
    as in the reference's python/engine/llm.py:18-30); -1 if the file or the key is missing."""
    path = Path(model_dir) / "generation_config.json"
    if not path.is_file():
        return -1
    try:
        raw = json.loads(path.read_text(encoding="utf-8"))
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: invalid JSON: {e}") from e
    return end_token_of(raw) if isinstance(raw, dict) else -1


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
