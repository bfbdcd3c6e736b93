"""Feed-forward parts.  ``DenseFeedForward``: ``down(act(up(x)))``, no gate, no experts
(``FalconMLP`` src/transformers/models/falcon/modeling_falcon.py:565-578).  The activation is one of the
reference's by name (src/transformers/activations.py:200-220; ``gelu`` is the exact erf form, :59-78), applied
in 32-bit in the epilogue of the first product."""
from __future__ import annotations

from typing import Sequence

import torch

from .. import ops
from .base import Part, StepContext, as_tensor, register_part
from .linear import Linear, PendingProjection


class DenseFeedForward(Part):
    def __init__(self, name: str, hidden_size: int, ffn_size: int, bias: bool, activation: str = "gelu",
                 up_name: str = "dense_h_to_4h", down_name: str = "dense_4h_to_h"):
        if activation not in ops.ACT_CODES:
            raise ValueError(f"activation {activation!r} is not built; built: {sorted(k for k in ops.ACT_CODES if k)}")
        self.name = name
        self.activation = activation
        self.up = Linear(f"{name}.{up_name}", hidden_size, ffn_size, bias)
        self.down = Linear(f"{name}.{down_name}", ffn_size, hidden_size, bias)

    def children(self) -> Sequence[Part]:
        return (self.up, self.down)

    can_defer = True

    def input_projection(self):
        """The first product of ``forward`` and how it is called (see ``AttentionMixer.input_projection``)."""
        return self.up, {"act": self.activation}

    def forward(self, x: torch.Tensor, ctx: StepContext, add1=None, add2=None, defer: bool = False, projected=None):
        """``down(act(up(x))) + add1 + add2``.  With ``defer`` the second product comes back not run
        (``PendingProjection``) and the caller sees to the additions."""
        h = projected if projected is not None else self.up(x, act=self.activation)
        if defer:
            return PendingProjection(self.down, h)
        return self.down(h, add1=as_tensor(add1), add2=as_tensor(add2))


register_part("feed_forward", "dense", DenseFeedForward)
