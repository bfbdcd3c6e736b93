"""Logits processors and the next-token choice."""
from .sampler import Sampler, philox_uniform

__all__ = ["Sampler", "philox_uniform"]
