"""Matrix products of the parts, with the normalisation of their input folded in where the
kernel can do it.

A norm part may hand its consumer a LazyNorm instead of a normalised tensor: the float32 residual
stream, the norm weight and eps.  `linear()` gives it to the fused kernel when that takes the
shape (bfloat16, few rows) and otherwise normalises first, so a part written against `linear()`
never needs to know which happened.  Parts that want a plain tensor call `materialize()`.

Between two layers the norm can also be started by the product before it: `linear(..., then_norm=
norm)` on a product that adds into the residual stream returns ScaledRows when the kernel took it
(bfloat16, at most 16 rows: decoding), which the next `linear()` completes in its epilogue.  That
saves the norm kernel between every two products of a decode step.
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


@dataclass
class ScaledRows:
    """An RMSNorm that the product before it began: x = bf16(h * norm weight) and partial sums of
    h^2 per row; the normalised rows are x[r] * rsqrt(sum_p sumsq[p, r] / size + eps)."""
    x: torch.Tensor                 # bf16 [count, size]
    sumsq: torch.Tensor             # float32 [parts, count]
    eps: float
    count: int

    def materialize(self, ctx) -> torch.Tensor:
        out = ctx.scratch("norm_out", (self.count, self.x.shape[1]), ctx.dtype)
        ops.scale_rows(out, self.x, self.sumsq, self.eps)
        return out


def materialize(ctx, x):
    return x.materialize(ctx) if isinstance(x, (LazyNorm, ScaledRows)) else x


def rows_of(x) -> int:
    return x.count if isinstance(x, (LazyNorm, ScaledRows)) else x.shape[0]


def _norm_ahead(ctx, then_norm, out, weight, m: int, accumulate: bool, swiglu: bool):
    """Buffers for the norm that follows a product, if the kernel can begin it: the norm must be
    an RMSNorm (it says so through `rms_parameters()`), the product must add into the residual."""
    parameters = getattr(then_norm, "rms_parameters", None)
    if parameters is None or not accumulate or swiglu or ctx.dtype != torch.bfloat16 or out.dtype != torch.float32:
        return None
    n, k = weight.shape
    if not ops.gemm_chains_norm(weight.dtype, m, k) or out.shape != (m, n):
        return None
    norm_weight, eps = parameters()
    if norm_weight.numel() != n:
        return None
    # two sets of buffers in turn: the one a product reads may not be the one it writes
    turn = ctx.memo["norm_ahead_turn"] = 1 - ctx.memo.get("norm_ahead_turn", 0)
    x = ctx.scratch(f"norm_ahead_x{turn}", (m, n), torch.bfloat16)
    sumsq = ctx.scratch(f"norm_ahead_sumsq{turn}", (ops.norm_chain_parts(n), m), torch.float32)
    return ScaledRows(x, sumsq, eps, m), norm_weight


def linear(ctx, out, x, weight, bias=None, accumulate: bool = False, swiglu: bool = False, then_norm=None):
    """out = x @ weight.T (+ bias), x a tensor, a LazyNorm or ScaledRows.

    then_norm: the norm part that will be applied to `out` next (only meaningful with
    `accumulate`).  Returns that norm of the updated `out` if it was computed on the way, as
    ScaledRows (begun by the few-rows kernel, finished by the next `linear()`) or as a plain
    tensor (after a library product); else None: the caller then runs the norm as usual.

    Products of more than 128 rows in bfloat16 go to the vendor's matrix library (as the reference's
    nn.Linear does) when the step allows it (`ctx.library_gemm`); its result then reaches the
    residual stream or the gated activation through one more small kernel.  Everything else,
    and every float32 product, runs in this package's own kernels (17..128 rows: the kernel that
    shares the activations through LDS, when the shape suits it: K a multiple of 256)."""
    scaled = None
    if isinstance(x, ScaledRows):
        if ops.gemm_chains_norm(weight.dtype, x.count, weight.shape[1]):
            scaled, x = x, x.x
        elif (ops.gemm_mid_takes(weight.dtype, x.count, weight.shape[0], weight.shape[1], ops.MID_ROWS_PREFERRED) and bias is None
              and not accumulate and out.dtype in (torch.bfloat16, torch.float32) and not (swiglu and out.dtype != torch.bfloat16)):
            # 17..128 rows: the product finishes the norm that the product before it began
            ops.gemm_mid_scaled(out, x.x, weight, x.sumsq, x.eps, swiglu)
            return None
        else:
            x = x.materialize(ctx)
    if not isinstance(x, LazyNorm) and x.dtype == torch.bfloat16:
        ahead = _norm_ahead(ctx, then_norm, out, weight, x.shape[0], accumulate, swiglu) if then_norm is not None else None
        if scaled is not None or ahead is not None:
            following, norm_weight = ahead if ahead is not None else (None, None)
            ops.gemm_norm_chain(out, x, weight, bias, accumulate, swiglu,
                                in_sumsq=None if scaled is None else scaled.sumsq, in_eps=0.0 if scaled is None else scaled.eps,
                                next_x=None if following is None else following.x,
                                next_sumsq=None if following is None else following.sumsq, next_weight=norm_weight)
            return following
    if isinstance(x, LazyNorm):
        if ops.gemm_fuses_norm(weight.dtype, x.count, weight.shape[1]) and ops.gemm_norm_fusion_pays(weight.shape[0]):
            ops.gemm(out, x.h, weight, bias, accumulate, swiglu, norm_weight=x.weight, eps=x.eps, rows=x.rows, count=x.count)
            return None
        x = x.materialize(ctx)
    m, n = x.shape[0], weight.shape[0]
    library = getattr(ctx, "library_gemm", False)
    # 17..128 rows: this package's kernel for them, whether or not the step may use the vendor library
    if (x.dtype == torch.bfloat16 and bias is None and x.is_contiguous() and (accumulate or out.dtype in (torch.bfloat16, torch.float32))
            and not (swiglu and out.dtype != torch.bfloat16)
            and ops.gemm_mid_takes(weight.dtype, m, n, weight.shape[1], ops.MID_ROWS_PREFERRED if library else 128)):
        parameters = getattr(then_norm, "rms_parameters", None) if accumulate else None
        if parameters is not None and out.is_contiguous() and out.dtype == torch.float32 and parameters()[0].numel() == n:
            # product, residual add and the first half of the norm that follows: the kernel that adds the K
            # splits' sums leaves bf16(h * norm weight) and partial sums of squares, the next product finishes
            norm_weight, eps = parameters()
            turn = ctx.memo["norm_ahead_turn"] = 1 - ctx.memo.get("norm_ahead_turn", 0)
            begun = ScaledRows(ctx.scratch(f"norm_ahead_x{turn}", (m, n), torch.bfloat16),
                               ctx.scratch(f"norm_begin_sumsq{turn}", (ops.norm_begin_parts(n), m), torch.float32), eps, m)
            ops.gemm_mid_add_norm_begin(out, x, weight, norm_weight, begun.x, begun.sumsq)
            return begun
        ops.gemm(out, x, weight, None, accumulate, swiglu)
        return None
    if (library and weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and m > ops.skinny_max_m()
            and bias is None and x.is_contiguous() and (accumulate or (out.dtype in (torch.bfloat16, torch.float32) and out.is_contiguous()))
            and not (swiglu and out.dtype != torch.bfloat16)):
        if accumulate or swiglu:
            y = ctx.scratch("library_gemm_out", (m, n), torch.bfloat16)
            torch.mm(x, weight.t(), out=y)
            if accumulate:
                parameters = getattr(then_norm, "rms_parameters", None)
                if parameters is not None and out.is_contiguous() and parameters()[0].numel() == n:
                    # the residual add and the norm that follows it in one pass over the rows
                    norm_weight, eps = parameters()
                    normed = ctx.scratch("norm_after_add", (m, n), ctx.dtype)
                    ops.add_rmsnorm(normed, out, y, norm_weight, eps)
                    return normed
                ops.add_into(out, y)
            else:
                ops.silu_mul(out, y, interleaved=True)
        elif out.dtype == torch.float32:
            torch.mm(x, weight.t(), out_dtype=torch.float32, out=out)     # float32 logits of many rows
        else:
            torch.mm(x, weight.t(), out=out)
        return None
    ops.gemm(out, x, weight, bias, accumulate, swiglu)
    return None
