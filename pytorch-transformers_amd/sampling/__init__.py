"""Logits processors and the next-token choice."""
from .ahead import TokensAhead
from .custom import LogitsProcessor, LogitsProcessorList, StoppingCriteria, StoppingCriteriaList
from .sampler import Sampler, philox_uniform

__all__ = ["LogitsProcessor", "LogitsProcessorList", "Sampler", "StoppingCriteria", "StoppingCriteriaList", "TokensAhead",
           "philox_uniform"]
