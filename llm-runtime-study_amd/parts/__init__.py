"""Parts a layer is composed of; importing this package registers the built-in kinds."""

from .base import (LazyTensors, PagedKVNeed, Part, PartSpec, StateNeed, TensorSpec, Under, create, register, under)
from . import attention, block, mlp, norm, rope  # noqa: F401  (registration)

__all__ = ["PagedKVNeed", "Part", "PartSpec", "StateNeed", "TensorSpec", "create", "register"]
