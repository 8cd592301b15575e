"""Typed configurations and the architecture registry."""

from .qwen3 import Qwen3Config
from .registry import (Architecture, ModelConfig, architecture_for, architecture_of, chat_template_for, config_from_dict,
                       load_config, register_architecture, registered_architectures, spec_for)

__all__ = ["Architecture", "ModelConfig", "Qwen3Config", "architecture_for", "architecture_of", "chat_template_for",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures", "spec_for"]
