"""One registry from the architecture's name (config.json ``architectures[0]``) to its typed
configuration and its model builder."""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Dict, Mapping, Type

from ..config.base import ConfigError, ModelConfig, read_config_json
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Type[ModelConfig]
    build: Callable[[ModelConfig], ModelSpec]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], build: Callable[[ModelConfig], ModelSpec]) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_cls, build)


def known_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def _ensure_builtin() -> None:
    from . import qwen2  # noqa: F401  (registers itself)


def architecture_of(raw: Mapping) -> Architecture:
    _ensure_builtin()
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, list):
        raise ConfigError("config.json: 'architectures' is missing; known architectures: "
                          + ", ".join(sorted(_ARCHITECTURES)))
    name = str(archs[0])
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config.json: architecture '{name}' is not registered; known: "
                          + ", ".join(sorted(_ARCHITECTURES)))
    return _ARCHITECTURES[name]


def parse_config(raw: Mapping) -> ModelConfig:
    return architecture_of(raw).config_cls.from_dict(raw)


def load_config(model_dir) -> ModelConfig:
    return parse_config(read_config_json(model_dir))


def build_model_spec(config: ModelConfig) -> ModelSpec:
    _ensure_builtin()
    if config.architecture not in _ARCHITECTURES:
        raise ConfigError(f"architecture '{config.architecture}' is not registered; known: "
                          + ", ".join(sorted(_ARCHITECTURES)))
    return _ARCHITECTURES[config.architecture].build(config)


def load_model(model_dir, dtype="bfloat16", device="cuda:0"):
    """The model of ``model_dir`` (config.json + model.safetensors) on the device."""
    from ..engine.model import Model

    return Model.from_pretrained(model_dir, dtype=dtype, device=device)
