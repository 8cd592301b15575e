"""Sampling parameters of one request (reference mini_llm/sampling.py:15-37)."""

from __future__ import annotations

import math
from dataclasses import dataclass

from ..errors import SamplingError


@dataclass(frozen=True)
class SamplingConfig:
    """temperature 0 picks the largest logit; a positive temperature draws from
    softmax(logits / temperature), optionally restricted by top-k and top-p."""

    temperature: float = 0.0
    top_k: int | None = None
    top_p: float = 1.0
    seed: int | None = None

    def __post_init__(self) -> None:
        if not math.isfinite(self.temperature) or self.temperature < 0:
            raise SamplingError("temperature must be finite and non-negative")
        if self.top_k is not None and self.top_k <= 0:
            raise SamplingError("top_k must be positive when supplied")
        if not math.isfinite(self.top_p) or not 0 < self.top_p <= 1:
            raise SamplingError("top_p must satisfy 0 < top_p <= 1")
        if self.seed is not None and self.seed < 0:
            raise SamplingError("seed must be non-negative when supplied")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0
