"""Typed configurations and the architecture registry."""

from .qwen3 import Qwen3Config
from .registry import (architecture_for, config_from_dict, load_config, register_architecture,
                       registered_architectures, spec_for)

__all__ = ["Qwen3Config", "architecture_for", "config_from_dict", "load_config", "register_architecture",
           "registered_architectures", "spec_for"]
