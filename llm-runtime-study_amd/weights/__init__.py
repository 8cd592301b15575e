"""Checkpoint reading, validation and random-weight generation."""

from .loader import load, validate
from .random_init import device_weights, random_tensors, write_model_dir
from .safetensors_io import Checkpoint, write_safetensors

__all__ = ["Checkpoint", "device_weights", "load", "random_tensors", "validate", "write_model_dir", "write_safetensors"]
