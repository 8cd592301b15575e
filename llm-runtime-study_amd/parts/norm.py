"""RMSNorm over the last dimension of the float32 residual stream.

Formula (reference mini_llm/nn/norm.py:42-46): y = w * x * rsqrt(mean(x^2) + eps), statistics
in float32.  The kernel rounds once, at the output, to the activation dtype.
"""

from __future__ import annotations

from ..kernels import ops
from .base import Part, TensorSpec, register
from .linear import LazyNorm


class RMSNorm(Part):
    graph_safe = True  # launches only library kernels on arena buffers
    plan_safe = True
    has_lazy_form = True

    def __init__(self, size: int, eps: float):
        if size <= 0:
            raise ValueError(f"size must be positive, got {size}")
        if eps <= 0:
            raise ValueError(f"eps must be positive, got {eps}")
        self.size, self.eps = size, eps
        self.weight = None

    def tensors(self):
        return {"weight": TensorSpec((self.size,), role="norm")}

    def bind(self, weights, dtype):
        self.weight = weights["weight"]

    def rms_parameters(self):
        """(weight, eps): says that this norm is w * x * rsqrt(mean(x^2) + eps), so that the matrix
        product before it may begin it (see parts/linear.py)."""
        return self.weight, self.eps

    def forward(self, ctx, h, rows=None, count=None, lazy: bool = False):
        """Normalise rows of h [*, size] (all, or the `count` rows listed in `rows`).

        With `lazy` the work is left to the consumer's matrix product (see parts/linear.py)."""
        n = h.shape[0] if rows is None else count
        pending = LazyNorm(h, self.weight, self.eps, rows, n)
        return pending if lazy else pending.materialize(ctx)


register("norm", "rmsnorm", RMSNorm)
