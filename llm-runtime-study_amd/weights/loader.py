"""Checks a checkpoint against the tensors a model asks for, then loads them by name.

All problems are collected and raised as one error before any tensor data is read
(reference mini_llm/checkpoint.py:453-487, call order mini_llm/model/base.py:279-291):
missing tensors, unexpected tensors, wrong shapes, and dtypes that cannot hold the role.
Floating tensors keep their stored precision on the way to the device (bfloat16 stays
bfloat16, 32-bit stays 32-bit; float16, which no kernel takes, is widened to float32);
integer tables become int32.
"""

from __future__ import annotations

from typing import Mapping

import torch

from ..errors import CheckpointValidationError
from ..parts import TensorSpec
from .safetensors_io import Checkpoint

FLOAT_DTYPES = ("F32", "BF16", "F16")
INT_DTYPES = ("I64", "I32", "I16", "I8", "U8")


def validate(checkpoint: Checkpoint, expected: Mapping[str, TensorSpec], architecture: str) -> None:
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
        allowed = INT_DTYPES if spec.dtype == "int32" else FLOAT_DTYPES
        if info.dtype not in allowed:
            errors.append(f"dtype mismatch for {name}: expected one of {', '.join(allowed)}, got {info.dtype}")
    if errors:
        raise CheckpointValidationError(
            f"checkpoint does not match {architecture} configuration:\n  - " + "\n  - ".join(errors))


def load(checkpoint: Checkpoint, expected: Mapping[str, TensorSpec], architecture: str, device) -> dict[str, torch.Tensor]:
    """Validate, then move every expected tensor that is present to `device`."""
    validate(checkpoint, expected, architecture)
    out = {}
    for name, spec in expected.items():
        if name not in checkpoint.manifest:
            continue
        t = checkpoint.tensor(name)
        if spec.dtype == "int32":
            t = t.to(torch.int32)
        elif t.dtype == torch.float16:
            t = t.to(torch.float32)
        out[name] = t.to(device)
    return out
