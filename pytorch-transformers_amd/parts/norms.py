"""Norms.  ``LayerNorm``: mean and biased variance over the features, affine always
(``torch.nn.LayerNorm`` as built at src/transformers/models/falcon/modeling_falcon.py:603-612, :843)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..engine.spec import INIT_ONE_NOISE, INIT_ZERO_NOISE, VECTOR, TensorSpec
from .base import Part, ResidualSum, register_part


class LayerNorm(Part):
    def __init__(self, name: str, hidden_size: int, eps: float):
        self.name = name
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.hidden_size,), VECTOR, INIT_ONE_NOISE),
                TensorSpec(self.name + ".bias", (self.hidden_size,), VECTOR, INIT_ZERO_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name + ".weight"]
        self.bias = tensors[self.name + ".bias"]

    def _wide_loads(self, x: torch.Tensor) -> bool:
        # bfloat16 rows of a width the sixteen-byte kernel takes: the one that also forms residual sums
        return x.dtype == torch.bfloat16 and ops.layernorm_sum_ok(self.hidden_size)

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self._wide_loads(x):
            return ops.layernorm_sum([x], self.hidden_size, w=self.weight, b=self.bias, eps=self.eps, rows=rows,
                                     want_x=False)[1]
        return ops.layernorm(x, self.weight, self.bias, self.eps, rows=rows)

    def forward_pair(self, x: torch.Tensor, other: "Part"):
        """``(self(x), other(x))``; one pass over x when both are LayerNorms with one eps."""
        if isinstance(other, LayerNorm) and other.eps == self.eps:
            if self._wide_loads(x):
                return ops.layernorm_sum([x], self.hidden_size, w=self.weight, b=self.bias, eps=self.eps,
                                         w2=other.weight, b2=other.bias, want_x=False)[1:]
            return ops.layernorm(x, self.weight, self.bias, self.eps, w2=other.weight, b2=other.bias)
        return self.forward(x), other.forward(x)


    def forward_sum(self, total: ResidualSum, rows: Optional[torch.Tensor] = None, other: Optional["Part"] = None,
                    want_x: bool = True):
        """``(x, self(x), other(x))`` for the unformed sum ``total``: x is formed, rounded and normalised in
        one pass.  Falls back to forming the sum first where the fused kernel does not take the width."""
        pair = isinstance(other, LayerNorm) and other.eps == self.eps
        if total.features == self.hidden_size and ops.layernorm_sum_ok(self.hidden_size) and (other is None or pair):
            return ops.layernorm_sum(total.kernel_terms(), self.hidden_size, w=self.weight, b=self.bias, eps=self.eps,
                                     w2=other.weight if pair else None, b2=other.bias if pair else None, rows=rows,
                                     want_x=want_x)
        x = total.tensor()
        if other is None:
            return x, self.forward(x, rows=rows), None
        a, m = self.forward_pair(x, other)
        return x, a, m


register_part("norm", "layernorm", LayerNorm)
