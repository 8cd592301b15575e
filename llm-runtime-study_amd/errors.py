"""Typed errors of the runtime; the command line maps each to `error: ...` and exit code 2."""


class ConfigError(ValueError):
    """A model configuration is missing, malformed or inconsistent."""


class CheckpointError(ValueError):
    """A checkpoint cannot be read."""


class CheckpointValidationError(CheckpointError):
    """Checkpoint contents do not match the tensors the model expects."""


class KVCacheError(ValueError):
    """Cache pages, slots or positions are invalid or exhausted."""


class GenerationError(ValueError):
    """A generation request cannot be executed."""


class SamplingError(ValueError):
    """Sampling parameters or logits are invalid."""


class EngineError(ValueError):
    """A device, dtype or context length is unsupported."""


class TokenizerError(ValueError):
    """Tokenizer files are missing or inconsistent with the model."""


class KernelError(RuntimeError):
    """The HIP kernel library is missing, failed to build, or refused its operands."""
