"""Interfaces of the parts a layer is put together from, and the registry that builds them.

A part is created from plain parameters (sizes and constants, never a model configuration),
then told which tensors it wants (`tensors()`), then given them (`bind()`).  It never learns
which model it is in.  Kinds are looked up by name in one registry per role, so a test or a
new architecture adds a kind with `register(role, name, cls)` and nothing else changes.

Roles and what each must provide:

  norm           forward(ctx, h, rows=None, count=None) -> x    h float32 [T, H] -> activation dtype; with `rows`
                                                        (int32 on the device) only the `count` rows listed there
  position       tables(ctx) -> (cos, sin) | None       float32 [T, rot/2] for this step's tokens
  mixer          cache_need() -> PagedKVNeed | StateNeed | None
                 forward(ctx, x, residual, cache)       adds its output into residual (float32)
  feed_forward   forward(ctx, x, residual)              adds its output into residual (float32)
  block          forward(ctx, h, cache)                 one layer: norms, mixer, feed-forward
  transform      forward(ctx, x)                        works in place on float32 rows: the residual stream [T, H] right
                                                        after the embedding (ModelSpec.after_embedding: a position signal
                                                        added there, a scale), or the logits [wanted, V] (ModelSpec.after_head:
                                                        a scale, a soft cap).  ctx.positions / ctx.logit_rows say which
                                                        tokens the rows belong to

Optional, each announced by a class attribute (a part without it is simply given plain tensors):

  has_lazy_form = True        norm: forward(..., lazy=True) may return a description of the norm (LazyNorm of
                              parts/linear.py) instead of a tensor; asked for only when the consumer takes one
  takes_lazy_norm = True      mixer / feed_forward: `x` may be a description of the norm (LazyNorm or
                              ScaledRows of parts/linear.py) that its first `linear()` completes
  begins_next_norm = True     mixer / feed_forward: forward(..., then_norm=norm) may return ScaledRows,
                              the norm of the updated residual begun by its last product, or None
  chains_norms = True         block: forward(ctx, h, cache, normed=None, then_norm=None) takes the
                              normalised input a previous block began and may return the next one;
                              `first_norm` is the norm it applies to its input

  wants_query_groups = True   mixer (a block passes it on): the step function cuts the tokens of a ragged step into
                              query groups for it: ctx.qblock_token0 / ctx.qblock_count [ctx.num_qblocks] list groups of
                              at most ctx.max_qblock consecutive tokens of one request, longest context first, which
                              together cover every token once.  In a step that is not decode-only the requests at its
                              head that bring one token each (ctx.single_rows of them; their tokens are the step's
                              first rows) are left out of the groups, which count their tokens from the first row
                              after them: a mixer that uses the groups serves those single rows itself (attention
                              gives them to its kernel for decode steps).  Without the attribute nothing is built and
                              ctx.num_qblocks is 0: a model of other mixers does not pay for it

A part may also say how its steps can be run again without it (both default to no):

  graph_safe = True           it launches only kernels on preallocated buffers, and reads the step's data from
                              the device (never from ctx.host_*): decode steps can be captured in a HIP graph
  plan_safe = True            it launches through this package's kernels (kernels/ops.py) alone, with arguments that
                              follow from the step's shape: a step's launches can be recorded and made again by
                              one call (engine/step.py), without running the part

`ctx` is the StepContext of engine/step.py: the step's token metadata on the device and a
scratch arena.  The residual stream `h` is float32 in every precision mode.
"""

from __future__ import annotations

import math
from collections.abc import Mapping as MappingView
from dataclasses import dataclass, field
from typing import Any, Callable, Iterable, Mapping

import torch

ROLES = ("norm", "position", "mixer", "feed_forward", "block", "transform")
_REGISTRY: dict[str, dict[str, type]] = {role: {} for role in ROLES}


def register(role: str, kind: str, cls: type) -> None:
    """Make `kind` available for `role`; registering a name twice replaces it."""
    if role not in _REGISTRY:
        raise KeyError(f"unknown part role {role!r}; roles are {ROLES}")
    _REGISTRY[role][kind] = cls


def create(role: str, spec: "PartSpec"):
    """Build the part that `spec` names, passing its parameters as keyword arguments."""
    try:
        cls = _REGISTRY[role][spec.kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRY.get(role, {}))) or "none"
        raise KeyError(f"no {role} of kind {spec.kind!r} is registered (known: {known})") from None
    return cls(**spec.params)


class LazyTensors(MappingView):
    """Tensors by name, each made when it is asked for (and again at every asking: nothing is kept here).  A
    model whose parts take their tensors one after the other then never holds a second copy of all its weights:
    the raw tensor of a matrix lives only while the part that asked for it puts it into its own form."""

    def __init__(self, names: Iterable[str], make: Callable[[str], torch.Tensor]):
        self._names, self._make = tuple(names), make
        self._known = frozenset(self._names)

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._known:
            raise KeyError(name)
        return self._make(name)

    def __iter__(self):
        return iter(self._names)

    def __len__(self) -> int:
        return len(self._names)

    def __contains__(self, name) -> bool:
        return name in self._known


class Under(MappingView):
    """The tensors of `weights` whose names begin with `prefix`, under the rest of their names.  A view: nothing
    is looked up before it is asked for, so tensors that are made on demand (LazyTensors) stay so."""

    def __init__(self, weights: Mapping[str, torch.Tensor], prefix: str):
        self._weights, self._prefix = weights, prefix

    def __getitem__(self, name: str) -> torch.Tensor:
        return self._weights[self._prefix + name]

    def __iter__(self):
        cut = len(self._prefix)
        return (name[cut:] for name in self._weights if name.startswith(self._prefix))

    def __len__(self) -> int:
        return sum(1 for _ in self)

    def __contains__(self, name) -> bool:
        return isinstance(name, str) and self._prefix + name in self._weights


def under(weights: Mapping[str, torch.Tensor], prefix: str) -> Mapping[str, torch.Tensor]:
    """What a part that owns the names under `prefix` is given to bind()."""
    return Under(weights, prefix)


@dataclass(frozen=True)
class PartSpec:
    """Kind and parameters of one part, as data."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class TensorSpec:
    """Shape and role of one checkpoint tensor a part wants.

    role: "matrix" ([out, in] projection), "embedding", "norm" (scale around 1), "bias";
    the random-weights mode draws each role differently.  dtype "float" follows the
    checkpoint (bfloat16 stays bfloat16, a tensor stored in 32-bit stays so); "int32"
    marks integer tables.
    """

    shape: tuple[int, ...]
    role: str = "matrix"
    dtype: str = "float"
    optional: bool = False


@dataclass(frozen=True)
class PagedKVNeed:
    """A mixer that keeps keys and values of every position (or of a window) in pages; `dtype`: what the pages
    hold, if not the run's activation dtype."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None
    dtype: torch.dtype | None = None


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a state of fixed size per request."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    """Common behaviour: a part owns no tensor until bind() hands it the ones it asked for."""

    def tensors(self) -> dict[str, TensorSpec]:
        return {}

    def bind(self, weights: Mapping[str, torch.Tensor], dtype: torch.dtype) -> None:
        """Take the device tensors named by tensors(); `dtype` is the activation dtype."""

    def weight_bytes(self) -> int:
        """Bytes of weights that one step reads (for roofline accounting)."""
        return 0

    def flops(self, tokens: int, pairs: int) -> float:
        """Floating-point operations of this part's matrix products in a step of `tokens` tokens (for roofline
        accounting; elementwise work is left out).  `pairs` is the number of (query, earlier-or-same position)
        pairs of the step under a causal mask: tokens * (tokens + 1) / 2 for a prompt read from its start, the
        sum of the context lengths for decoding requests.  Only mixers that look back use it.  Unless a part says
        otherwise: every matrix it declares in tensors() is multiplied with every token once."""
        return 2.0 * tokens * sum(math.prod(spec.shape) for spec in self.tensors().values() if spec.role == "matrix")


def flops_of(part, tokens: int, pairs: int) -> float:
    """part.flops(tokens, pairs), also for a part that does not derive from Part and says nothing of its own
    (then: its declared matrices, each multiplied with every token once)."""
    own = getattr(part, "flops", None)
    return own(tokens, pairs) if own is not None else Part.flops(part, tokens, pairs)


def length_class(length: int) -> int:
    """`length` rounded down to 256 times a power of two (0 below 256). Choices that follow the
    context length (how far decode attention is split) are made per class, so that eager steps and
    graph replays agree bit for bit and a growing context recaptures a handful of times."""
    blocks = length // 256
    return 256 << (blocks.bit_length() - 1) if blocks else 0
