"""Rotary position encoding with half-split pairs (i, i + rot/2).

Reference mini_llm/nn/rope.py:34-40 (inverse frequencies 1 / theta^(2i/d) in float32),
74-80 (angle = float32(position) * inv_freq), 110-146 (rotation).  The tables are made once
per step, in float32, and shared by every layer that uses this encoding; the rotation itself
is fused into the attention mixer's q/k kernel.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, register


class RotaryHalfSplit(Part):
    def __init__(self, rotary_dim: int, theta: float):
        if rotary_dim <= 0 or rotary_dim % 2 != 0:
            raise ValueError(f"rotary_dim must be a positive even integer, got {rotary_dim}")
        if theta <= 0:
            raise ValueError(f"theta must be positive, got {theta}")
        self.rotary_dim, self.theta = rotary_dim, theta
        dims = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
        self._inv_freq_host = 1.0 / (theta ** (dims / rotary_dim))
        self._inv_freq = None

    def key(self):
        return ("rope_half", self.rotary_dim, self.theta)

    def tables(self, ctx):
        """cos and sin [T, rotary_dim/2] float32 for this step's positions (made once per step)."""
        cached = ctx.memo.get(self.key())
        if cached is None:
            if self._inv_freq is None or self._inv_freq.device != ctx.positions.device:
                self._inv_freq = self._inv_freq_host.to(ctx.positions.device)
            half = self.rotary_dim // 2
            cos = ctx.scratch(f"rope_cos_{self.rotary_dim}_{self.theta}", (ctx.T, half), torch.float32)
            sin = ctx.scratch(f"rope_sin_{self.rotary_dim}_{self.theta}", (ctx.T, half), torch.float32)
            ops.rope_table(cos, sin, ctx.positions, self._inv_freq)
            cached = ctx.memo[self.key()] = (cos, sin)
        return cached


class NoPosition(Part):
    """No position signal inside the mixer."""

    def tables(self, ctx):
        return None


register("position", "rope_half", RotaryHalfSplit)
register("position", "none", NoPosition)
