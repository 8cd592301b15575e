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
    """out = x @ weight.T (+ bias), x a tensor or a LazyNorm.

    Products of many rows in bfloat16 go to the vendor's matrix library (as the reference's
    nn.Linear does) when the step allows it (`ctx.library_gemm`); its result then reaches the
    residual stream or the gated activation through one more small kernel.  Everything else,
    and every float32 product, runs in this package's own kernels."""
    if isinstance(x, LazyNorm):
        if ops.gemm_fuses_norm(weight.dtype, x.count, weight.shape[1]) and ops.gemm_norm_fusion_pays(weight.shape[0]):
            ops.gemm(out, x.h, weight, bias, accumulate, swiglu, norm_weight=x.weight, eps=x.eps, rows=x.rows, count=x.count)
            return
        x = x.materialize(ctx)
    m, n = x.shape[0], weight.shape[0]
    if (getattr(ctx, "library_gemm", False) and weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and m > ops.skinny_max_m()
            and bias is None and x.is_contiguous() and (accumulate or (out.dtype == torch.bfloat16 and out.is_contiguous()))):
        if accumulate or swiglu:
            y = ctx.scratch("library_gemm_out", (m, n), torch.bfloat16)
            torch.mm(x, weight.t(), out=y)
            if accumulate:
                ops.add_into(out, y)
            else:
                ops.silu_mul(out, y, interleaved=True)
        else:
            torch.mm(x, weight.t(), out=out)
        return
    ops.gemm(out, x, weight, bias, accumulate, swiglu)
