"""From a model folder (or a configuration and a seed) to a bound model on the device."""

from __future__ import annotations

import math

import torch

from ..config import load_config, spec_for
from ..errors import EngineError
from ..models import DecoderModel
from ..parts import LazyTensors
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


# One piece of device memory for all that an engine holds
#
# Every large tensor that torch allocates by itself is a mapping of its own, and the device translates addresses in
# such a mapping through page-table entries of 2 MB.  One allocation of many gigabytes is mapped with far larger
# entries, and the kernels of a decode step, each of which begins by touching weights no kernel before it has touched,
# miss the translation caches less: measured on the MI355X at the 8B sizes, 4.00 -> 3.95 ms a step at batch 8 and
# 3.74 -> 3.70 ms at batch 1 (nothing at 0.6B).  So before an engine's weights are made, one tensor of about the size of
# everything the engine will hold is allocated and given back: torch's caching allocator keeps the segment and cuts the
# weights, the cache pool and the step's buffers out of it.  Nothing depends on that happening: an allocator that
# works otherwise (caching switched off, expandable segments) leaves the engine as it was without this.
RESERVE_AT_LEAST = 1 << 30        # smaller engines are a few mappings anyway
RESERVE_MARGIN = 3 << 29          # the step's buffers (activations, logits, metadata) beside weights and cache


def engine_bytes(model: DecoderModel, dtype: torch.dtype, page_size: int, num_pages: int) -> int:
    """About how many bytes of device memory an engine of `model` (bound or not) holds: its weights in `dtype`
    and its cache pool of `num_pages` pages; an estimate (integer tables and 32-bit norms count as `dtype`)."""
    from ..parts import PagedKVNeed, StateNeed

    item = torch.empty(0, dtype=dtype).element_size()
    total = sum(math.prod(spec.shape) for spec in model.tensors().values()) * item
    for need in model.cache_needs():
        if isinstance(need, PagedKVNeed):
            size = item if need.dtype is None else torch.empty(0, dtype=need.dtype).element_size()
            total += 2 * need.num_kv_heads * need.head_dim * size * page_size * (num_pages + 1)
        elif isinstance(need, StateNeed):
            total += math.prod(need.shape) * torch.empty(0, dtype=need.dtype).element_size()
    return total


def reserve_device_memory(num_bytes: int, device) -> int:
    """Allocate one tensor of `num_bytes` and a margin (in whole gigabytes) and give it back to torch's allocator,
    which keeps the segment for the allocations that follow.  Returns the bytes reserved (0: nothing; an allocation
    that does not fit fails cleanly)."""
    if num_bytes < RESERVE_AT_LEAST:
        return 0
    num_bytes = -(-(num_bytes + RESERVE_MARGIN) >> 30) << 30
    try:
        slab = torch.empty(num_bytes, dtype=torch.uint8, device=device)
    except torch.OutOfMemoryError:
        return 0
    del slab
    return num_bytes


def reserve_for(config, dtype: torch.dtype, device, page_size: int, num_pages: int) -> int:
    """reserve_device_memory() for an engine of `config` that is about to be made.  The device is initialised before
    the engine's size is worked out, not by the allocation itself right after it: measured several times over on the
    MI355X, a process whose first use of the device was followed at once by this allocation ran its decode steps 0.5 %
    slower than one with a few tenths of a second of host work between the two (3.95 against 3.93 ms); why is not known."""
    torch.cuda.init()
    return reserve_device_memory(engine_bytes(DecoderModel(spec_for(config)), dtype, page_size, num_pages), device)


def load_model(model_dir, dtype: torch.dtype, device, config=None, stored_precision: bool = False) -> tuple:
    """(typed configuration, bound DecoderModel) of a model folder.

    The checkpoint's floating tensors must be stored in the configuration's dtype, as in the reference
    (mini_llm/checkpoint.py:478-481); `stored_precision=True` takes them in whatever floating dtype they
    are stored (a bfloat16 model with 32-bit norm weights, say) and keeps that precision."""
    config = load_config(model_dir) if config is None else config
    spec = spec_for(config)
    model = DecoderModel(spec)
    checkpoint = Checkpoint.from_model_dir(model_dir)
    # validated as a whole first; then every tensor is read and moved when its part asks for it
    weights = load(checkpoint, model.tensors(), config.model_type, device, None if stored_precision else spec.checkpoint_dtype, lazy=True)
    try:
        model.bind(weights, dtype)
    finally:
        checkpoint.close()
    return config, model


def random_model(config, seed: int, dtype: torch.dtype, device, init: str = "normal") -> DecoderModel:
    """Bound model with random weights made on the device (no files)."""
    spec = spec_for(config)
    model = DecoderModel(spec)
    # drawn in the precision the architecture's checkpoints are stored in, and brought to the device as a loaded
    # checkpoint is: float16, which no kernel takes, widened to float32
    drawn = device_weights(model, seed, TORCH_DTYPES[spec.checkpoint_dtype], device, init)

    def widened(name: str) -> torch.Tensor:
        t = drawn[name]
        return t.float() if t.dtype == torch.float16 else t

    model.bind(LazyTensors(list(drawn), widened), dtype)
    return model
