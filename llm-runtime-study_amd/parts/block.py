"""Arrangement of norms, mixer and feed-forward in one layer.

PreNormBlock (reference mini_llm/model/qwen.py:58-72):
    h = h + mixer(norm1(h));  h = h + feed_forward(norm2(h))
The two sums happen inside the parts, which add into the float32 residual stream.
"""

from __future__ import annotations

from .base import Part, PartSpec, create, flops_of, register, under
from .linear import materialize


class PreNormBlock(Part):
    def __init__(self, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec, ff_norm: PartSpec,
                 names: dict | None = None):
        self.mixer = create("mixer", mixer)
        self.feed_forward = create("feed_forward", feed_forward)
        self.mixer_norm = create("norm", mixer_norm)
        self.ff_norm = create("norm", ff_norm)
        self.names = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "mixer_norm", "ff_norm": "ff_norm"}
        self.names.update(names or {})

    def _children(self):
        return [(self.names[k], getattr(self, k)) for k in ("mixer_norm", "mixer", "ff_norm", "feed_forward")]

    def tensors(self):
        return {f"{prefix}.{name}": spec for prefix, part in self._children() for name, spec in part.tensors().items()}

    def bind(self, weights, dtype):
        for prefix, part in self._children():
            part.bind(under(weights, prefix + "."), dtype)

    def weight_bytes(self):
        return sum(part.weight_bytes() for _, part in self._children())

    def flops(self, tokens, pairs):
        return sum(flops_of(part, tokens, pairs) for _, part in self._children())

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._children())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(part, "plan_safe", False) for _, part in self._children())

    @property
    def wants_query_groups(self) -> bool:
        return getattr(self.mixer, "wants_query_groups", False)

    chains_norms = True

    @property
    def first_norm(self):
        return self.mixer_norm

    def forward(self, ctx, h, cache, normed=None, then_norm=None):
        """Run the layer on the residual stream h.  `normed`: this layer's first norm of h, already
        begun by the product that last updated h; `then_norm`: the norm that follows this layer.
        Returns that norm of the updated h if the last product began it, else None."""
        # a consumer that says `takes_lazy_norm` gets the norm as a description to fold into its
        # first matrix product; any other gets the normalised tensor
        x = self._normed(ctx, self.mixer_norm, self.mixer, h, normed)
        if getattr(self.mixer, "begins_next_norm", False):
            begun = self.mixer.forward(ctx, x, h, cache, then_norm=self.ff_norm)
        else:
            self.mixer.forward(ctx, x, h, cache)
            begun = None
        x = self._normed(ctx, self.ff_norm, self.feed_forward, h, begun)
        if then_norm is not None and getattr(self.feed_forward, "begins_next_norm", False):
            return self.feed_forward.forward(ctx, x, h, then_norm=then_norm)
        self.feed_forward.forward(ctx, x, h)
        return None

    @staticmethod
    def _normed(ctx, norm, consumer, h, begun=None):
        lazy = getattr(consumer, "takes_lazy_norm", False)
        if begun is not None:
            return begun if lazy else materialize(ctx, begun)
        if lazy and getattr(norm, "has_lazy_form", False):
            return norm.forward(ctx, h, lazy=True)
        return norm.forward(ctx, h)


register("block", "prenorm", PreNormBlock)
