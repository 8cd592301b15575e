"""Greedy, temperature, top-k, top-p and seeded sampling."""

from .config import SamplingConfig
from .sampler import Sampler, SamplingRow, request_seed

__all__ = ["Sampler", "SamplingConfig", "SamplingRow", "request_seed"]
