"""Checkpoint reading, validation and random-weight generation."""

from .loader import load, validate
from .safetensors_io import Checkpoint, write_safetensors

__all__ = ["Checkpoint", "device_weights", "load", "random_tensors", "validate", "write_model_dir", "write_safetensors"]

_RANDOM_INIT = ("device_weights", "random_tensors", "write_model_dir", "random_init")


def __getattr__(name):
    # random_init is also a program (`python -m ...weights.random_init`): importing it only when one of
    # its names is asked for keeps the interpreter from finding it loaded before it runs it
    if name in _RANDOM_INIT:
        from importlib import import_module
        module = import_module(".random_init", __name__)
        return module if name == "random_init" else getattr(module, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
