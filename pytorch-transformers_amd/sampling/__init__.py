"""Logits processors and the next-token choice."""
from .ahead import TokensAhead
from .sampler import Sampler, philox_uniform

__all__ = ["Sampler", "TokensAhead", "philox_uniform"]
