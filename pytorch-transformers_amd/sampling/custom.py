"""The containers for a caller's own processors and stopping criteria, as ``generate(logits_processor=...,
stopping_criteria=...)`` takes them (any list of callables does; these are the reference's names for them).

A processor is called as ``processor(input_ids, scores) -> scores`` and a criterion as ``criterion(input_ids,
scores) -> flags`` with ``input_ids`` int64 ``[rows, longest]`` (shorter rows padded on the left) and ``scores``
32-bit ``[rows, vocab]`` on the model's device (src/transformers/generation/logits_process.py:45-78,
stopping_criteria.py:46-57, :491-497).
"""
from __future__ import annotations

import torch


class LogitsProcessor:
    def __call__(self, input_ids: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError(f"{type(self).__name__} must define __call__(input_ids, scores) -> scores")


class StoppingCriteria:
    def __call__(self, input_ids: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError(f"{type(self).__name__} must define __call__(input_ids, scores) -> flags per row")


class LogitsProcessorList(list):
    """Processors applied one after the other (src/transformers/generation/logits_process.py:55-78)."""

    def __call__(self, input_ids: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
        for processor in self:
            scores = processor(input_ids, scores)
        return scores


class StoppingCriteriaList(list):
    """A row ends when any criterion says so (src/transformers/generation/stopping_criteria.py:491-497)."""

    def __call__(self, input_ids: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
        done = torch.zeros(input_ids.shape[0], dtype=torch.bool, device=input_ids.device)
        for criterion in self:
            said = criterion(input_ids, scores)
            done = done | (said if isinstance(said, torch.Tensor) else torch.tensor(bool(said), device=done.device))
        return done
