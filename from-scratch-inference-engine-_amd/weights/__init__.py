"""Weights: the safetensors file format, loading by tensor name, and seeded random weights."""

from .safetensors_file import SafetensorsError, SafetensorsFile, write_safetensors
from .loader import CheckpointFiles, ParamBinding, TensorSpec, WeightsError, load_weights
from .random_init import random_checkpoint_tensors, write_random_model

__all__ = ["CheckpointFiles", "ParamBinding", "SafetensorsError", "SafetensorsFile", "TensorSpec", "WeightsError",
           "load_weights", "random_checkpoint_tensors", "write_random_model", "write_safetensors"]
