"""Checks a checkpoint against the tensors a model asks for, then loads them by name.

All problems are collected and raised as one error before any tensor data is read
(reference mini_llm/checkpoint.py:453-487, call order mini_llm/model/base.py:279-291):
missing tensors, unexpected tensors, wrong shapes and wrong dtypes.

Which dtype a floating tensor must have follows the configuration, as in the reference
(mini_llm/checkpoint.py:39-43 maps `torch_dtype` to the container's dtype names, 478-481
reports a mismatch): `checkpoint_dtype` "bfloat16" wants BF16 and so on.  With
`checkpoint_dtype=None` (the explicit option of `load()` for folders of mixed precision,
which the replay tool uses) any floating dtype passes and the stored precision is kept.
Integer tables may come in any integer width.

On the way to the device floating tensors keep their stored precision: bfloat16 stays
bfloat16, 32-bit stays 32-bit; float16, which no kernel takes, is widened to float32 (exact);
integer tables become int32.
"""

from __future__ import annotations

from typing import Mapping

import torch

from ..errors import CheckpointValidationError
from ..parts import LazyTensors, TensorSpec
from .safetensors_io import Checkpoint

FLOAT_DTYPES = ("F32", "BF16", "F16")
INT_DTYPES = ("I64", "I32", "I16", "I8", "U8")
CONFIG_TO_CONTAINER_DTYPE = {"float16": "F16", "bfloat16": "BF16", "float32": "F32"}


def validate(checkpoint: Checkpoint, expected: Mapping[str, TensorSpec], architecture: str,
             checkpoint_dtype: str | None = None) -> None:
    """Raise one CheckpointValidationError that lists everything in which the checkpoint's manifest
    differs from `expected`.  checkpoint_dtype: the configuration's `torch_dtype`, which every
    floating tensor must then be stored in; None accepts any floating dtype."""
    if checkpoint_dtype is not None and checkpoint_dtype not in CONFIG_TO_CONTAINER_DTYPE:
        raise CheckpointValidationError(
            f"unsupported checkpoint dtype {checkpoint_dtype!r}; expected one of: {', '.join(sorted(CONFIG_TO_CONTAINER_DTYPE))}")
    wanted_float = None if checkpoint_dtype is None else CONFIG_TO_CONTAINER_DTYPE[checkpoint_dtype]
    actual = checkpoint.manifest
    required = {name for name, spec in expected.items() if not spec.optional}
    errors = []
    missing = sorted(required - actual.keys())
    unexpected = sorted(actual.keys() - expected.keys())
    if missing:
        errors.append("missing tensors: " + ", ".join(missing))
    if unexpected:
        errors.append("unexpected tensors: " + ", ".join(unexpected))
    for name in sorted(expected.keys() & actual.keys()):
        spec, info = expected[name], actual[name]
        if info.shape != tuple(spec.shape):
            errors.append(f"shape mismatch for {name}: expected {tuple(spec.shape)}, got {info.shape}")
        if spec.dtype == "int32":
            if info.dtype not in INT_DTYPES:
                errors.append(f"dtype mismatch for {name}: expected one of {', '.join(INT_DTYPES)}, got {info.dtype}")
        elif wanted_float is not None:
            if info.dtype != wanted_float:
                errors.append(f"dtype mismatch for {name}: expected {wanted_float}, got {info.dtype}")
        elif info.dtype not in FLOAT_DTYPES:
            errors.append(f"dtype mismatch for {name}: expected one of {', '.join(FLOAT_DTYPES)}, got {info.dtype}")
    if errors:
        raise CheckpointValidationError(
            f"checkpoint does not match {architecture} configuration:\n  - " + "\n  - ".join(errors))


def load(checkpoint: Checkpoint, expected: Mapping[str, TensorSpec], architecture: str, device,
         checkpoint_dtype: str | None = None, lazy: bool = False) -> Mapping[str, torch.Tensor]:
    """Validate (see validate() for `checkpoint_dtype`), then move every expected tensor that is
    present to `device` in its stored precision.  lazy: each tensor is read and moved when it is asked for
    (parts.LazyTensors; the checkpoint must stay open meanwhile), so that a model which takes its tensors part
    by part never holds the checkpoint and its own form of the weights at once."""
    validate(checkpoint, expected, architecture, checkpoint_dtype)

    def fetch(name: str) -> torch.Tensor:
        t = checkpoint.tensor(name)
        if expected[name].dtype == "int32":
            t = t.to(torch.int32)
        elif t.dtype == torch.float16:
            t = t.to(torch.float32)
        return t.to(device)

    present = [name for name in expected if name in checkpoint.manifest]
    return LazyTensors(present, fetch) if lazy else {name: fetch(name) for name in present}
