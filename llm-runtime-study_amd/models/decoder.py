"""Decoder-only language model assembled from a ModelSpec.

Embedding, the scheduled layers, final norm, LM head (reference mini_llm/model/base.py:72-89
for the stack, mini_llm/model/qwen.py:109-112 for the head; a tied head reuses the embedding
table).  The forward runs only the tokens of the step it is given, reading and writing the
caches that the step context carries; it holds no per-request state itself.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from ..parts import TensorSpec, create
from ..parts.base import flops_of, under
from ..parts.linear import linear
from .spec import ModelSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.layers = [create("block", block) for block in spec.layers]
        self.final_norm = create("norm", spec.final_norm)
        # optional parts around the stack: (part, prefix of its tensors' names)
        self.after_embedding = None if spec.after_embedding is None else create("transform", spec.after_embedding)
        self.after_head = None if spec.after_head is None else create("transform", spec.after_head)
        self.embedding = self.head = None
        self.dtype = None

    # ------------------------------------------------------------------ weights
    def tensors(self) -> dict[str, TensorSpec]:
        """Every checkpoint tensor by full name."""
        spec = self.spec
        out = {spec.embedding_name: TensorSpec((spec.vocab_size, spec.hidden_size), role="embedding")}
        for index, layer in enumerate(self.layers):
            prefix = spec.layer_prefix.format(index=index)
            out.update({f"{prefix}.{name}": t for name, t in layer.tensors().items()})
        out.update({f"{spec.final_norm_prefix}.{name}": t for name, t in self.final_norm.tensors().items()})
        for part, prefix in self._around():
            out.update({f"{prefix}.{name}": t for name, t in part.tensors().items()})
        out[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden_size), role="matrix", optional=spec.tie_head)
        return out

    def bind(self, weights: dict[str, torch.Tensor], dtype: torch.dtype) -> None:
        """Hand every part its tensors; `dtype` is the activation (and matrix) dtype of the run."""
        spec = self.spec
        self.dtype = dtype
        self.embedding = weights[spec.embedding_name].to(dtype).contiguous()
        head = weights.get(spec.head_name)
        self.head = self.embedding if head is None else head.to(dtype).contiguous()
        for index, layer in enumerate(self.layers):
            prefix = spec.layer_prefix.format(index=index) + "."
            layer.bind(under(weights, prefix), dtype)
        for part, prefix in [(self.final_norm, spec.final_norm_prefix)] + self._around():
            prefix += "."
            part.bind(under(weights, prefix), dtype)

    def _around(self) -> list:
        """The optional parts after the embedding and after the head, each with the prefix of its tensors."""
        return [(part, prefix) for part, prefix in ((self.after_embedding, self.spec.after_embedding_prefix),
                                                    (self.after_head, self.spec.after_head_prefix)) if part is not None]

    def _parts(self) -> list:
        return self.layers + [self.final_norm] + [part for part, _ in self._around()]

    def cache_needs(self) -> list:
        """What each schedule entry keeps between steps: a need, ("from", entry) or None."""
        needs = []
        for entry in self.spec.schedule:
            if entry.cache_from is not None:
                needs.append(("from", entry.cache_from))
            else:
                needs.append(self.layers[entry.layer].cache_need())
        return needs

    def graph_safe(self) -> bool:
        """Whether a step launches only this library's kernels on preallocated buffers, so that it
        can be captured in a HIP graph: every part must say so itself."""
        return all(getattr(part, "graph_safe", False) for part in self._parts())

    def wants_query_groups(self) -> bool:
        """Whether any mixer reads the step's query groups (see parts/base.py); the step function builds them only then."""
        return any(getattr(layer, "wants_query_groups", False) for layer in self.layers)

    def plan_safe(self) -> bool:
        """Whether a step's launches can be written down once and made again from the record: every part must
        launch through this package's kernels alone, with arguments that follow from the step's shape."""
        return all(getattr(part, "plan_safe", False) for part in self._parts())

    def weight_bytes(self, with_embedding: bool = False) -> int:
        """Bytes of weights one decode step reads: every scheduled layer once, and the head."""
        total = sum(self.layers[e.layer].weight_bytes() for e in self.spec.schedule)
        total += sum(part.weight_bytes() for part, _ in self._around())
        total += self.head.numel() * self.head.element_size()
        if with_embedding and self.head is not self.embedding:
            total += self.embedding.numel() * self.embedding.element_size()
        return total

    def flops(self, tokens: int, pairs: int, logit_rows: int = 1) -> float:
        """Floating-point operations of the matrix products of one step of `tokens` tokens: every scheduled layer
        (what each part says of itself, see Part.flops for `pairs`) and the head for `logit_rows` rows."""
        total = sum(flops_of(self.layers[e.layer], tokens, pairs) for e in self.spec.schedule)
        total += sum(flops_of(part, tokens, pairs) for part, _ in self._around())
        return total + 2.0 * logit_rows * self.spec.vocab_size * self.spec.hidden_size

    # ------------------------------------------------------------------ forward
    def forward_hidden(self, ctx) -> torch.Tensor:
        """Residual stream [T, H] float32 after the last layer (before the final norm)."""
        h = ctx.scratch("residual", (ctx.T, self.spec.hidden_size), torch.float32)
        ops.embed(h, self.embedding, ctx.token_ids, self.spec.embedding_multiplier)
        if self.after_embedding is not None:
            self.after_embedding.forward(ctx, h)
        schedule = self.spec.schedule
        begun = None   # the next layer's first norm, if the product that last updated h began it
        for position, entry in enumerate(schedule):
            layer = self.layers[entry.layer]
            if not getattr(layer, "chains_norms", False):
                layer.forward(ctx, h, ctx.layer_cache(position))
                begun = None
                continue
            following = self.layers[schedule[position + 1].layer] if position + 1 < len(schedule) else None
            then_norm = following.first_norm if getattr(following, "chains_norms", False) else None
            begun = layer.forward(ctx, h, ctx.layer_cache(position), normed=begun, then_norm=then_norm)
        return h

    def logits(self, ctx, h: torch.Tensor) -> torch.Tensor:
        """float32 logits [n_wanted, V] at the rows of `h` listed in ctx.logit_rows."""
        n = ctx.num_logit_rows
        if getattr(self.final_norm, "has_lazy_form", False):   # the head's product normalises its own input
            x = self.final_norm.forward(ctx, h, rows=ctx.logit_rows, count=n, lazy=True)
        else:
            x = self.final_norm.forward(ctx, h, rows=ctx.logit_rows, count=n)
        out = ctx.scratch("logits", (n, self.spec.vocab_size), torch.float32)
        linear(ctx, out, x, self.head)
        if self.after_head is not None:
            self.after_head.forward(ctx, out)
        return out
