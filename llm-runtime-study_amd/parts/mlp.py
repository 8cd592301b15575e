"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), three bias-free projections.

Reference mini_llm/nn/mlp.py:80-87.  gate and up are stacked into one [2I, H] matrix when
the weights are bound, so one product feeds the gated activation; the down projection adds
straight into the float32 residual stream.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, TensorSpec, register
from .linear import linear, rows_of


class SwiGLU(Part):
    graph_safe = True  # launches only library kernels on arena buffers
    plan_safe = True
    takes_lazy_norm = True
    begins_next_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        if hidden_size <= 0 or intermediate_size <= 0:
            raise ValueError("hidden_size and intermediate_size must be positive")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.gate_up = self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": TensorSpec((i, h)),
            "up_proj.weight": TensorSpec((i, h)),
            "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, weights, dtype):
        gate, up = weights["gate_proj.weight"].to(dtype), weights["up_proj.weight"].to(dtype)
        h, i = self.hidden_size, self.intermediate_size
        # bfloat16: rows interleaved in groups of 8 (8 gate rows, then the 8 up rows of the same
        # features), so that the product's epilogue has both halves of a feature and writes
        # silu(gate) * up itself; otherwise gate rows then up rows and a separate activation kernel
        self.interleaved = dtype == torch.bfloat16 and i % 8 == 0 and h % 8 == 0
        if self.interleaved:
            self.gate_up = torch.stack((gate.view(i // 8, 8, h), up.view(i // 8, 8, h)), 1).reshape(2 * i, h).contiguous()
        else:
            self.gate_up = torch.cat((gate, up), 0).contiguous()
        self.down = weights["down_proj.weight"].to(dtype).contiguous()

    def weight_bytes(self):
        return (self.gate_up.numel() + self.down.numel()) * self.down.element_size()

    def forward(self, ctx, x, residual, then_norm=None):
        t = rows_of(x)
        act = ctx.scratch("ffn_act", (t, self.intermediate_size), ctx.dtype)
        if self.interleaved:
            linear(ctx, act, x, self.gate_up, swiglu=True)
        else:
            gate_up = ctx.scratch("ffn_gate_up", (t, 2 * self.intermediate_size), ctx.dtype)
            linear(ctx, gate_up, x, self.gate_up)
            ops.silu_mul(act, gate_up)
        return linear(ctx, residual, act, self.down, accumulate=True, then_norm=then_norm)


register("feed_forward", "swiglu", SwiGLU)
