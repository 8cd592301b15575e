"""MI355X-native one-GPU inference runtime for Qwen3 dense models.

    from llm_runtime_study_amd import Engine, SamplingConfig
    engine = Engine.from_model_dir("model_dir", max_batch_size=8)
    for index, event in engine.generate([[1, 2, 3]], max_new_tokens=16):
        ...
"""

from .errors import (CheckpointError, CheckpointValidationError, ConfigError, EngineError, GenerationError,
                     KernelError, KVCacheError, SamplingError, TokenizerError)
from .sampling.config import SamplingConfig
from .text.chat import ChatMessage

__all__ = ["ChatMessage", "CheckpointError", "CheckpointValidationError", "ConfigError", "Engine", "EngineError",
           "GenerationError", "GenerationEvent", "KVCacheError", "KernelError", "Qwen3Config", "SamplingConfig",
           "SamplingError", "TokenizerError", "load_config"]


def __getattr__(name):
    # the engine pulls in torch and the kernel library; load it on first use
    if name == "Engine":
        from .engine.engine import Engine
        return Engine
    if name == "GenerationEvent":
        from .engine.scheduler import GenerationEvent
        return GenerationEvent
    if name in ("Qwen3Config", "load_config"):       # as the reference's package exports them (mini_llm/__init__.py)
        from . import config
        return getattr(config, name)
    raise AttributeError(name)
