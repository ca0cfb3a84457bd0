"""Architectures: one module each, registered by the name config.json gives."""

from .registry import (architecture_of, build_model_spec, known_architectures, load_config, load_model,
                       parse_config, register_architecture)
from .spec import LayerCall, ModelSpec, bind

__all__ = ["LayerCall", "ModelSpec", "architecture_of", "bind", "build_model_spec", "known_architectures",
           "load_config", "load_model", "parse_config", "register_architecture"]
