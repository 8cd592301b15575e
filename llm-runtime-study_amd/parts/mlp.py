"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), three bias-free projections.

Reference mini_llm/nn/mlp.py:80-87.  gate and up are stacked into one [2I, H] matrix when
the weights are bound, so one product feeds the gated activation; the down projection adds
straight into the float32 residual stream.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, TensorSpec, register


class SwiGLU(Part):
    graph_safe = True  # launches only library kernels on arena buffers

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
        self.gate_up = torch.cat((weights["gate_proj.weight"], weights["up_proj.weight"]), 0).to(dtype).contiguous()
        self.down = weights["down_proj.weight"].to(dtype).contiguous()

    def weight_bytes(self):
        return (self.gate_up.numel() + self.down.numel()) * self.down.element_size()

    def forward(self, ctx, x, residual):
        t = x.shape[0]
        gate_up = ctx.scratch("ffn_gate_up", (t, 2 * self.intermediate_size), ctx.dtype)
        ops.gemm(gate_up, x, self.gate_up)
        act = ctx.scratch("ffn_act", (t, self.intermediate_size), ctx.dtype)
        ops.silu_mul(act, gate_up)
        ops.gemm(residual, act, self.down, accumulate=True)


register("feed_forward", "swiglu", SwiGLU)
