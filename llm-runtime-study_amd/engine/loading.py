"""From a model folder (or a configuration and a seed) to a bound model on the device."""

from __future__ import annotations

import torch

from ..config import load_config, spec_for
from ..errors import EngineError
from ..models import DecoderModel
from ..weights import Checkpoint, device_weights, load
from ..weights.random_init import TORCH_DTYPES

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def resolve_device(requested="auto") -> torch.device:
    """The GPU to run on.  There is no CPU path: a missing GPU is an error.

    Reference mini_llm/engine.py:70-103 resolves cpu/mps/cuda; this runtime runs on the
    HIP device only (torch names it "cuda").
    """
    if requested in ("auto", "cuda", "hip"):
        requested = "cuda"
    try:
        device = torch.device(requested)
    except (TypeError, RuntimeError) as exc:
        raise EngineError(f"invalid device {requested!r}") from exc
    if device.type != "cuda":
        raise EngineError(f"unsupported device {device}; this runtime runs on the GPU only (use 'cuda' or 'auto')")
    if not torch.cuda.is_available():
        raise EngineError("a GPU was requested but none is available")
    if device.index is not None and device.index >= torch.cuda.device_count():
        raise EngineError(f"GPU index {device.index} is unavailable; found {torch.cuda.device_count()} device(s)")
    return torch.device("cuda", device.index or 0)


def resolve_dtype(requested="auto") -> torch.dtype:
    """bfloat16 unless float32 is asked for (reference mini_llm/engine.py:106-132 defaults to
    float16 on accelerators; float16 is not a precision of this runtime)."""
    if requested == "auto":
        return torch.bfloat16
    if isinstance(requested, torch.dtype) and requested in DTYPES.values():
        return requested
    if isinstance(requested, str) and requested in DTYPES:
        return DTYPES[requested]
    raise EngineError(f"unsupported dtype {requested!r}; expected auto, {', '.join(DTYPES)}")


def load_model(model_dir, dtype: torch.dtype, device, config=None, stored_precision: bool = False) -> tuple:
    """(typed configuration, bound DecoderModel) of a model folder.

    The checkpoint's floating tensors must be stored in the configuration's dtype, as in the reference
    (mini_llm/checkpoint.py:478-481); `stored_precision=True` takes them in whatever floating dtype they
    are stored (a bfloat16 model with 32-bit norm weights, say) and keeps that precision."""
    config = load_config(model_dir) if config is None else config
    spec = spec_for(config)
    model = DecoderModel(spec)
    checkpoint = Checkpoint.from_model_dir(model_dir)
    weights = load(checkpoint, model.tensors(), config.model_type, device, None if stored_precision else spec.checkpoint_dtype)
    checkpoint.close()
    model.bind(weights, dtype)
    return config, model


def random_model(config, seed: int, dtype: torch.dtype, device, init: str = "normal") -> DecoderModel:
    """Bound model with random weights made on the device (no files)."""
    spec = spec_for(config)
    model = DecoderModel(spec)
    # drawn in the precision the architecture's checkpoints are stored in, and brought to the device as a loaded
    # checkpoint is: float16, which no kernel takes, widened to float32
    weights = device_weights(model, seed, TORCH_DTYPES[spec.checkpoint_dtype], device, init)
    model.bind({name: t.float() if t.dtype == torch.float16 else t for name, t in weights.items()}, dtype)
    return model
