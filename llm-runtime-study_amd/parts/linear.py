"""Matrix products of the parts, with the normalisation of their input folded in where the
kernel can do it.

A norm part may hand its consumer a LazyNorm instead of a normalised tensor: the float32 residual
stream, the norm weight and eps.  `linear()` gives it to the fused kernel when that takes the
shape (bfloat16, few rows) and otherwise normalises first, so a part written against `linear()`
never needs to know which happened.  Parts that want a plain tensor call `materialize()`.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import ops


@dataclass
class LazyNorm:
    h: torch.Tensor                 # float32 [*, size]
    weight: torch.Tensor
    eps: float
    rows: torch.Tensor | None       # int32 rows of h to take, or None for the first `count`
    count: int

    def materialize(self, ctx) -> torch.Tensor:
        out = ctx.scratch("norm_out", (self.count, self.h.shape[1]), ctx.dtype)
        ops.rmsnorm(out, self.h, self.weight, self.eps, rows=self.rows)
        return out


def materialize(ctx, x):
    return x.materialize(ctx) if isinstance(x, LazyNorm) else x


def rows_of(x) -> int:
    return x.count if isinstance(x, LazyNorm) else x.shape[0]


def linear(ctx, out, x, weight, bias=None, accumulate: bool = False, swiglu: bool = False) -> None:
    """out = x @ weight.T (+ bias), x a tensor or a LazyNorm."""
    if isinstance(x, LazyNorm):
        if ops.gemm_fuses_norm(weight.dtype, x.count, weight.shape[1]):
            ops.gemm(out, x.h, weight, bias, accumulate, swiglu, norm_weight=x.weight, eps=x.eps, rows=x.rows, count=x.count)
            return
        x = x.materialize(ctx)
    ops.gemm(out, x, weight, bias, accumulate, swiglu)
