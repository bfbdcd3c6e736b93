"""Position encodings: what rotates queries and keys, and what is added to attention scores."""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from .base import Part, register_part


class NoPositions(Part):
    def to(self, device) -> None:
        pass

    def rotation(self) -> Tuple[Optional[torch.Tensor], float]:
        return None, 1.0

    def score_bias(self) -> Optional[torch.Tensor]:
        return None


class RotaryPositions(NoPositions):
    """Rotation of element pairs ``(i, i + d/2)`` by ``position * inv_freq[i]``.

    ``inv_freq[i] = 1 / theta^(2i/d)`` in 32-bit
    (src/transformers/modeling_rope_utils.py:58-68); linear scaling divides it by ``factor``
    (:108).  Angles, cosines and sines are 32-bit in the kernel, as the reference forces them
    to be (src/transformers/models/falcon/modeling_falcon.py:155-164).
    """

    def __init__(self, head_dim: int, theta: float, scaling_factor: float = 1.0, attention_scaling: float = 1.0):
        if head_dim % 2:
            raise ValueError(f"rotary positions need an even head size, got {head_dim}")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.scaling_factor = float(scaling_factor)
        self.attention_scaling = float(attention_scaling)
        inv = 1.0 / (self.theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
        if self.scaling_factor != 1.0:
            inv = inv / self.scaling_factor
        self.inv_freq = inv.contiguous()

    def to(self, device) -> None:
        self.inv_freq = self.inv_freq.to(device)

    def rotation(self):
        return self.inv_freq, self.attention_scaling


def alibi_slopes(num_heads: int) -> torch.Tensor:
    """Per-head slopes, 32-bit values (src/transformers/models/falcon/modeling_falcon.py:173-188)."""
    n2 = 2 ** math.floor(math.log2(num_heads))
    base = torch.tensor(2 ** (-(2 ** -(math.log2(n2) - 3))), dtype=torch.float32)
    slopes = torch.pow(base, torch.arange(1, 1 + n2, dtype=torch.int32))
    if n2 != num_heads:
        extra_base = torch.tensor(2 ** (-(2 ** -(math.log2(2 * n2) - 3))), dtype=torch.float32)
        remaining = min(n2, num_heads - n2)
        extra = torch.pow(extra_base, torch.arange(1, 1 + 2 * remaining, 2, dtype=torch.int32))
        slopes = torch.cat([slopes, extra], dim=0)
    return slopes


class AlibiPositions(NoPositions):
    """A bias ``slope_h * key position`` on the scores, nothing on queries and keys.

    The reference multiplies the slopes, rounded to bfloat16, by the position in bfloat16
    arithmetic whatever the model's type is
    (src/transformers/models/falcon/modeling_falcon.py:196-198) and divides by ``sqrt(d)`` when
    it folds the bias into the mask (:1078-1085).  The slopes are held here already rounded; the
    attention kernels round the position and the product.
    """

    def __init__(self, num_heads: int):
        self.num_heads = num_heads
        self.slopes = alibi_slopes(num_heads).bfloat16().float().contiguous()

    def to(self, device) -> None:
        self.slopes = self.slopes.to(device)

    def score_bias(self):
        return self.slopes


register_part("positions", "none", NoPositions)
register_part("positions", "rotary", RotaryPositions)
register_part("positions", "alibi", AlibiPositions)
