"""Tokens that a step chose and the host has not looked at yet.

A decode step is short, and between two of them the host waits for the chosen tokens, decides who goes on and
launches the next step: some hundred microseconds in which the GPU has nothing to do.  The tokens of a step are
therefore left on the device and the next step is launched from them at once; the host reads them while that step
runs, and a sequence that turns out to have ended took part in one step whose result nobody reads.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


class TokensAhead:
    """One token per row of a step, on the device (int32), on its way to pinned host memory."""

    def __init__(self, tensor: torch.Tensor):
        self.tensor = tensor
        self._host = torch.empty(tensor.shape, dtype=tensor.dtype, pin_memory=True)
        self._host.copy_(tensor, non_blocking=True)
        self._arrived = torch.cuda.Event()
        self._arrived.record()
        self._list: Optional[List[int]] = None
        #: the rows that the next step takes, in its order (None: all of them, in order)
        self.rows: Optional[Sequence[int]] = None

    def __len__(self) -> int:
        return int(self.tensor.shape[0])

    def take(self, rows: Optional[Sequence[int]]) -> "TokensAhead":
        """The same tokens, of which the next step is to take ``rows`` (indices, in the step's order)."""
        self.rows = None if rows is None or list(rows) == list(range(len(self))) else [int(r) for r in rows]
        return self

    def tolist(self) -> List[int]:
        """All rows' tokens; waits until they have arrived."""
        if self._list is None:
            self._arrived.synchronize()
            self._list = self._host.tolist()
        return self._list

    def for_step(self) -> torch.Tensor:
        """The tokens of ``rows`` as a device tensor, without a wait on the host."""
        if self.rows is None:
            return self.tensor
        idx = torch.tensor(self.rows, dtype=torch.int64).pin_memory().to(self.tensor.device, non_blocking=True)
        return self.tensor.index_select(0, idx)
