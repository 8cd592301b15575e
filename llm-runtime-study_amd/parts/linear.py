"""Matrix products of the parts, with the normalisation of their input folded in where the
kernel can do it.

A norm part may hand its consumer a LazyNorm instead of a normalised tensor: the float32 residual
stream, the norm weight and eps.  `linear()` gives it to the fused kernel when that takes the
shape (bfloat16, few rows) and otherwise normalises first, so a part written against `linear()`
never needs to know which happened.  Parts that want a plain tensor call `materialize()`.

Between two layers the norm can also be started by the product before it: `linear(..., then_norm=
norm)` on a product that adds into the residual stream returns ScaledRows when the kernel took it
(bfloat16, at most 128 rows: decoding), which the next `linear()` completes in its epilogue.  That
saves the norm kernel between every two products of a decode step.

Which kernel serves a product is decided in one place, `plan()`, from the product's shape, the
dtypes, the form its input arrives in and the step's KernelChoice (`ctx.kernels`); it returns the
name of a route and `linear()` runs it.  The routes:

  chain      at most 16 bfloat16 rows: the few-rows kernel finishing a norm begun before it and / or
             beginning the one that follows (gemm_norm_chain)
  mid_scaled 17..128 rows whose norm was begun before: the kernel for them finishes it (gemm_mid_scaled)
  fused_norm few rows of the float32 residual stream, normalised on the way in (gemm with norm_weight)
  mid_begin  17..128 rows adding into the residual stream and beginning the norm that follows
  mid        17..128 rows, nothing folded in (gemm picks the kernel for them)
  split_norm more than 128 rows adding into the residual stream before an RMSNorm, of a shape whose K this package's
             many-rows kernel divides between workgroups: the kernel that adds up their sums also adds the residual
             and normalises the rows (gemm_lines_add_rmsnorm)
  library    more rows than these kernels are made for, if the step may use the vendor library; the
             residual add (with the norm that follows) or the gated activation take one more small kernel
  own        everything else, and every float32 product (gemm picks the kernel by shape)
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


def kernels_of(ctx) -> ops.KernelChoice:
    return getattr(ctx, "kernels", None) or ops.DEFAULT_CHOICE


def workspace_of(ctx) -> tuple:
    """The step's own memory for the sums of products that divide K between workgroups (one per scratch arena, so two
    runners on two streams never share one)."""
    memo = getattr(ctx, "memo", None)
    known = None if memo is None else memo.get("gemm_workspace")
    if known is None:
        known = ops.workspace_address(ctx.scratch("gemm_split_sums", (ops.gemm_workspace_bytes() // 4,), torch.float32))
        if memo is not None:
            memo["gemm_workspace"] = known
    return known


ROUTES = ("chain", "mid_scaled", "fused_norm", "mid_begin", "mid", "split_norm", "library", "own")


def plan(m: int, n: int, k: int, *, weight_dtype: torch.dtype, run_dtype: torch.dtype, out_dtype: torch.dtype, arrives: str,
         accumulate: bool = False, swiglu: bool = False, bias: bool = False, norm_follows: int = 0,
         contiguous: bool = True, out_contiguous: bool = True, choice: ops.KernelChoice = ops.DEFAULT_CHOICE) -> tuple[str, str]:
    """(route, what to do with the input first) for out [m, n] = x [m, k] @ w[n, k].T.

    arrives: "tensor" (activation dtype), "lazy" (LazyNorm) or "scaled" (ScaledRows); norm_follows: the size
    of the RMSNorm the caller will apply to `out` next (0: none, or not an RMSNorm).  The second value says
    whether the input has to be turned into a plain tensor before the route runs: "" or "materialize"."""
    bf16 = weight_dtype == torch.bfloat16 and run_dtype == torch.bfloat16
    stores = out_dtype in (torch.bfloat16, torch.float32) and not (swiglu and out_dtype != torch.bfloat16)
    follows = bool(norm_follows) and norm_follows == n and accumulate and not swiglu and out_dtype == torch.float32
    if arrives == "scaled":
        if ops.gemm_chains_norm(weight_dtype, m, k, choice):
            return "chain", ""
        if ops.gemm_mid_takes(weight_dtype, m, n, k, ops.MID_ROWS_PREFERRED, choice) and not bias and not accumulate and stores:
            return "mid_scaled", ""
        arrives, first = "tensor", "materialize"
    elif arrives == "lazy":
        if ops.gemm_fuses_norm(weight_dtype, m, k, choice) and ops.gemm_norm_fusion_pays(n):
            return "fused_norm", ""
        arrives, first = "tensor", "materialize"
    else:
        first = ""
    if bf16 and follows and ops.gemm_chains_norm(weight_dtype, m, k, choice):
        return "chain", first
    mid_most = ops.MID_ROWS_PREFERRED if choice.library else 128
    if (bf16 and not bias and contiguous and (accumulate or stores)
            and ops.gemm_mid_takes(weight_dtype, m, n, k, mid_most, choice)):
        return ("mid_begin" if follows and out_contiguous else "mid"), first
    if (choice.library and bf16 and m > choice.few_rows_max and not bias and contiguous
            and (accumulate or (stores and out_contiguous))):
        if m > 128 and out_contiguous and ops.gemm_split_pays(m, n, k):
            # too few tiles for the chip and a long K: divided between workgroups here
            return ("split_norm" if follows and n % 4 == 0 and n <= 8192 else "own"), first
        return "library", first
    return "own", first


def _next_norm(then_norm, n: int):
    """(weight, eps) of the norm that follows if it is an RMSNorm over n columns (it says so through
    `rms_parameters()`), else None."""
    parameters = getattr(then_norm, "rms_parameters", None)
    if parameters is None:
        return None
    weight, eps = parameters()
    return (weight, eps) if weight.numel() == n else None


def _ahead_buffers(ctx, m: int, n: int, parts: int, eps: float, tag: str) -> ScaledRows:
    # two sets of buffers in turn: the one a product reads may not be the one it writes
    turn = ctx.memo["norm_ahead_turn"] = 1 - ctx.memo.get("norm_ahead_turn", 0)
    return ScaledRows(ctx.scratch(f"norm_ahead_x{turn}", (m, n), torch.bfloat16),
                      ctx.scratch(f"{tag}{turn}", (parts, m), torch.float32), eps, m)


def linear(ctx, out, x, weight, bias=None, accumulate: bool = False, swiglu: bool = False, then_norm=None):
    """out = x @ weight.T (+ bias), x a tensor, a LazyNorm or ScaledRows.

    then_norm: the norm part that will be applied to `out` next (only meaningful with
    `accumulate`).  Returns that norm of the updated `out` if it was computed on the way, as
    ScaledRows (begun by the product, finished by the next `linear()`) or as a plain tensor (after a
    library product); else None: the caller then runs the norm as usual."""
    choice = kernels_of(ctx)
    n, k = weight.shape
    m = rows_of(x)
    following = _next_norm(then_norm, n) if then_norm is not None and accumulate else None
    arrives = "scaled" if isinstance(x, ScaledRows) else "lazy" if isinstance(x, LazyNorm) else "tensor"
    route, first = plan(m, n, k, weight_dtype=weight.dtype, run_dtype=ctx.dtype, out_dtype=out.dtype, arrives=arrives,
                        accumulate=accumulate, swiglu=swiglu, bias=bias is not None, norm_follows=n if following else 0,
                        contiguous=arrives != "tensor" or x.is_contiguous(), out_contiguous=out.is_contiguous(), choice=choice)
    scaled = x if arrives == "scaled" and not first else None
    if first:
        x = x.materialize(ctx)
        # a plain tensor now: its dtype and layout may send it elsewhere than was planned for the norm's own form
        if route in ("mid", "mid_begin", "library", "split_norm") and not (x.dtype == torch.bfloat16 and x.is_contiguous()):
            route = "own"
    elif arrives == "tensor" and route != "own" and x.dtype != torch.bfloat16:
        route = "own"

    if route == "chain":
        begun = None
        if following is not None and not swiglu and out.dtype == torch.float32 and out.shape == (m, n):
            begun = _ahead_buffers(ctx, m, n, ops.norm_chain_parts(n), following[1], "norm_ahead_sumsq")
        ops.gemm_norm_chain(out, x.x if scaled is not None else x, weight, bias, accumulate, swiglu,
                            in_sumsq=None if scaled is None else scaled.sumsq, in_eps=0.0 if scaled is None else scaled.eps,
                            next_x=None if begun is None else begun.x, next_sumsq=None if begun is None else begun.sumsq,
                            next_weight=None if begun is None else following[0], choice=choice)
        return begun
    if route == "mid_scaled":
        ops.gemm_mid_scaled(out, scaled.x, weight, scaled.sumsq, scaled.eps, swiglu, choice=choice, workspace=workspace_of(ctx))
        return None
    if route == "fused_norm":
        ops.gemm(out, x.h, weight, bias, accumulate, swiglu, norm_weight=x.weight, eps=x.eps, rows=x.rows, count=x.count, choice=choice)
        return None
    if route == "mid_begin":
        # product, residual add and the first half of the norm that follows: the kernel that adds the K splits'
        # sums leaves bf16(h * norm weight) and partial sums of squares, the next product finishes
        begun = _ahead_buffers(ctx, m, n, ops.norm_begin_parts(n), following[1], "norm_begin_sumsq")
        ops.gemm_mid_add_norm_begin(out, x, weight, following[0], begun.x, begun.sumsq, choice=choice, workspace=workspace_of(ctx))
        return begun
    if route == "split_norm":
        normed = ctx.scratch("norm_after_add", (m, n), ctx.dtype)
        ops.gemm_lines_add_rmsnorm(out, x, weight, following[0], following[1], normed, workspace=workspace_of(ctx))
        return normed
    if route == "library":
        if not (accumulate or swiglu):
            ops.library_gemm(out, x, weight)                      # bfloat16, or the float32 logits of many rows
            return None
        y = ctx.scratch("library_gemm_out", (m, n), torch.bfloat16)
        ops.library_gemm(y, x, weight)
        if swiglu:
            ops.silu_mul(out, y, interleaved=True)
            return None
        if following is not None and out.is_contiguous():
            # the residual add and the norm that follows it in one pass over the rows
            normed = ctx.scratch("norm_after_add", (m, n), ctx.dtype)
            ops.add_rmsnorm(normed, out, y, following[0], following[1])
            return normed
        ops.add_into(out, y)
        return None
    # "mid" and "own": gemm picks the kernel by shape
    ops.gemm(out, x, weight, bias, accumulate, swiglu, choice=choice, workspace=workspace_of(ctx) if ctx.dtype == torch.bfloat16 else None)
    return None
