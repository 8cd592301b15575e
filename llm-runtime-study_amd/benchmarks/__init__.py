"""Workloads that measure the engine: layer shapes of the Qwen3 dense family and the staggered serving run."""

from .shapes import QWEN3_8B, SHAPES

__all__ = ["QWEN3_8B", "SHAPES"]
