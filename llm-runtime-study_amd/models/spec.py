"""Architecture-neutral description of a decoder model, as data.

An architecture turns its typed configuration into a ModelSpec; everything after that
(weights, cache groups, the step) reads the ModelSpec and never the architecture.

  layers    the distinct layers (each owns weights), described by a block PartSpec
  schedule  the order in which layers run: ScheduleEntry(layer, cache_from).  A layer may be
            named twice (same weights, a cache of its own for each run), and an entry may
            read the cache that an earlier entry writes (`cache_from` = index into schedule).
  after_embedding, after_head
            optional parts of the role "transform" that work in place on the float32 residual
            stream right after the embedding (a learned or absolute position signal, a scale)
            and on the float32 logits (a scale, a soft cap); their tensors are named
            `<after_embedding_prefix>.<name>` and `<after_head_prefix>.<name>`.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts import PartSpec


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple[PartSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    max_positions: int
    eos_token_ids: tuple[int, ...] = ()
    bos_token_id: int | None = None
    tie_head: bool = False
    embedding_multiplier: float = 1.0
    embedding_name: str = "model.embed_tokens.weight"
    head_name: str = "lm_head.weight"
    final_norm_prefix: str = "model.norm"
    layer_prefix: str = "model.layers.{index}"
    checkpoint_dtype: str = "bfloat16"
    after_embedding: PartSpec | None = None
    after_head: PartSpec | None = None
    after_embedding_prefix: str = "model.after_embedding"
    after_head_prefix: str = "after_head"
    extra: dict = field(default_factory=dict, compare=False)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for position, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule entry {position} names layer {entry.layer}, but there are {len(self.layers)} layers")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < position:
                    raise ValueError(f"schedule entry {position} may only read the cache of an earlier entry, got {entry.cache_from}")
                if self.schedule[entry.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {position} reads entry {entry.cache_from}, which owns no cache itself")
