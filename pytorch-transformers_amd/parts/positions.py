"""Position encodings: what rotates queries and keys, and what is added to attention scores.

Both are data that the kernels take (``Rotation``, ``ScoreBias``); a position encoding is a part that hands them
out.  Another scheme of either kind that the fields can say (a rotation of part of the head, interleaved pairs,
other frequencies; slopes times the distance instead of the key's position, another scale) is a new part and no
change to a kernel.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional, Tuple, Union

import torch

from .base import Part, register_part


@dataclasses.dataclass
class Rotation:
    """Queries and keys are rotated by position: the first ``rotary_dim`` elements of a head (None: all) in pairs
    ``(i, i + rotary_dim / 2)`` (``"half"``) or ``(2i, 2i + 1)`` (``"interleaved"``), pair i by the angle
    ``position * inv_freq[i]``, cosines and sines multiplied by ``scale``.  ``inv_freq`` is ``[rotary_dim / 2]``, or
    one such row per sequence of the step."""

    inv_freq: torch.Tensor
    scale: float = 1.0
    rotary_dim: Optional[int] = None
    pairing: str = "half"


@dataclasses.dataclass
class ScoreBias:
    """``slopes[head] * x * scale`` is added to the score of a query and a key: x is the key's position (``of="key"``)
    or the key's position minus the query's (``"distance"``).  ``bf16``: the position and the product are rounded to
    bfloat16 before the scale, and the slopes are held rounded (what the reference does, ``"key"`` only)."""

    slopes: torch.Tensor
    of: str = "key"
    bf16: bool = False
    scale: float = 1.0


def as_rotation(given) -> Optional[Rotation]:
    """What a position encoding's ``rotation()`` may return, as a ``Rotation`` or None: a ``Rotation``, None, or the
    pair ``(inv_freq or None, scale)`` of a rotation of whole heads in half-split pairs."""
    if given is None or isinstance(given, Rotation):
        return given
    inv_freq, scale = given
    return None if inv_freq is None else Rotation(inv_freq, float(scale))


def as_score_bias(given, head_dim: int) -> Optional[ScoreBias]:
    """What ``score_bias()`` may return, as a ``ScoreBias`` or None: a ``ScoreBias``, None, or a tensor of slopes per
    head, which stands for the reference's ALiBi (times the key's position, rounded to bfloat16, divided by the root
    of the head size; src/transformers/models/falcon/modeling_falcon.py:196-198, :1078-1085)."""
    if given is None or isinstance(given, ScoreBias):
        return given
    return ScoreBias(given, "key", True, 1.0 / math.sqrt(head_dim))


class NoPositions(Part):
    def to(self, device) -> None:
        pass

    def rotation(self) -> Union[None, Rotation, Tuple[Optional[torch.Tensor], float]]:
        return None

    def score_bias(self) -> Union[None, ScoreBias, torch.Tensor]:
        return None


class RotaryPositions(NoPositions):
    """Rotation of element pairs ``(i, i + d/2)`` by ``position * inv_freq[i]``.

    ``inv_freq[i] = 1 / theta^(2i/d)`` in 32-bit
    (src/transformers/modeling_rope_utils.py:58-68); linear scaling divides it by ``factor``
    (:108).  Angles, cosines and sines are 32-bit in the kernel, as the reference forces them
    to be (src/transformers/models/falcon/modeling_falcon.py:155-164).
    """

    def __init__(self, head_dim: int, theta: float, scaling_factor: float = 1.0, attention_scaling: float = 1.0,
                 inv_freq: Optional[torch.Tensor] = None, dynamic_factor: Optional[float] = None,
                 trained_positions: Optional[int] = None):
        """``inv_freq`` given: a table of ``head_dim / 2`` frequencies of another scheme (``yarn_frequencies``,
        ``llama3_frequencies``, ``longrope_frequencies``); cosines and sines are multiplied by
        ``attention_scaling`` (src/transformers/models/falcon/modeling_falcon.py:162-166).

        ``dynamic_factor`` with ``trained_positions``: dynamic NTK scaling
        (src/transformers/modeling_rope_utils.py:112-160).  The frequencies of a sequence follow its own length:
        up to ``trained_positions`` tokens they are the trained ones, beyond that those of the base
        ``theta * (factor * length / trained - (factor - 1)) ** (d / (d - 2))``, taken anew in every step from
        the length the sequence has after it.  Keys already in the cache keep the rotation of the step that
        wrote them, as they do in the reference (:136-156 there rotates only what a forward pass is given).
        The reference takes one length for a whole padded batch, the longest, and keeps the largest it has seen
        until a call shorter than the trained context resets it (modeling_falcon.py:136-153); here each
        sequence has its own, so that its logits do not depend on what else is in the batch: a sequence alone
        gets what the reference gives a batch of one."""
        if head_dim % 2:
            raise ValueError(f"rotary positions need an even head size, got {head_dim}")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.scaling_factor = float(scaling_factor)
        self.attention_scaling = float(attention_scaling)
        self.dynamic_factor = None if dynamic_factor is None else float(dynamic_factor)
        self.trained_positions = None if trained_positions is None else int(trained_positions)
        if self.dynamic_factor is not None:
            if self.trained_positions is None or self.trained_positions <= 0 or self.dynamic_factor < 1.0 or head_dim <= 2:
                raise ValueError("dynamic frequencies need a factor >= 1, the trained context length and a head size "
                                 f"above 2 (factor {dynamic_factor}, context {trained_positions}, head size {head_dim})")
        if inv_freq is not None:
            if tuple(inv_freq.shape) != (head_dim // 2,):
                raise ValueError(f"a frequency table for head size {head_dim} has {head_dim // 2} entries, got "
                                 f"{tuple(inv_freq.shape)}")
            inv = inv_freq.to(torch.float32)
        else:
            inv = default_frequencies(head_dim, self.theta)
            if self.scaling_factor != 1.0:
                inv = inv / self.scaling_factor
        self.inv_freq = inv.contiguous()

    def to(self, device) -> None:
        self.inv_freq = self.inv_freq.to(device)

    def rotation(self) -> Rotation:
        return Rotation(self.inv_freq, self.attention_scaling)

    def rotation_for(self, ctx) -> Rotation:
        """The rotation for one step: the table, or with dynamic scaling one table per sequence of the step,
        ``[sequences, head_dim / 2]``, made once per step on the device from the step's own arrays (so a captured
        step makes it anew at every replay)."""
        if self.dynamic_factor is None:
            return self.rotation()
        from .. import ops

        key = ("rotary frequencies", id(self))
        table = ctx.extras.get(key)
        if table is None:
            table = ctx.extras[key] = ops.rope_dynamic_table(ctx.seq_start, ctx.cu_tokens, self.head_dim, self.theta,
                                                             self.dynamic_factor, self.trained_positions)
        return Rotation(table, self.attention_scaling)


def default_frequencies(head_dim: int, theta: float) -> torch.Tensor:
    """``1 / theta^(2i/d)`` in 32-bit (src/transformers/modeling_rope_utils.py:58-68)."""
    return 1.0 / (float(theta) ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))


def yarn_frequencies(head_dim: int, theta: float, factor: float, max_position_embeddings: int,
                     beta_fast: float = 32.0, beta_slow: float = 1.0, attention_factor: Optional[float] = None):
    """YaRN (src/transformers/modeling_rope_utils.py:163-239): frequencies that turn often within the trained
    context stay, those that turn less than once are divided by ``factor``, and a linear ramp over the pair
    index blends the two in between; returns (table, factor on cosines and sines)."""
    scale = 0.1 * math.log(factor) + 1.0 if attention_factor is None else float(attention_factor)
    half = head_dim // 2

    def pair_with_turns(turns: float) -> float:  # the pair index whose frequency makes `turns` turns in the context
        return head_dim * math.log(max_position_embeddings / (turns * 2 * math.pi)) / (2 * math.log(theta))

    low = max(math.floor(pair_with_turns(beta_fast)), 0)
    high = min(math.ceil(pair_with_turns(beta_slow)), head_dim - 1)
    if low == high:
        high += 0.001
    ramp = torch.clamp((torch.arange(half, dtype=torch.float32) - low) / (high - low), 0, 1)
    keep = 1.0 - ramp  # 1: the frequency as trained, 0: divided by the factor
    turns_per_pos = theta ** (torch.arange(0, head_dim, 2).float() / head_dim)
    inv = (1.0 / (factor * turns_per_pos)) * (1 - keep) + (1.0 / turns_per_pos) * keep
    return inv, scale


def llama3_frequencies(head_dim: int, theta: float, factor: float, low_freq_factor: float, high_freq_factor: float,
                       original_max_position_embeddings: int) -> torch.Tensor:
    """Llama 3.1's scheme (src/transformers/modeling_rope_utils.py:310-341): wavelengths beyond
    ``original / low_freq_factor`` are stretched by ``factor``, those under ``original / high_freq_factor`` stay,
    and in between the two are blended by where the wavelength lies."""
    inv = default_frequencies(head_dim, theta)
    wavelen = 2 * math.pi / inv
    long_from = original_max_position_embeddings / low_freq_factor
    short_to = original_max_position_embeddings / high_freq_factor
    out = torch.where(wavelen > long_from, inv / factor, inv)
    smooth = (original_max_position_embeddings / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    blended = (1 - smooth) * out / factor + smooth * out
    middle = ~(wavelen < short_to) & ~(wavelen > long_from)
    return torch.where(middle, blended, out)


def longrope_frequencies(head_dim: int, theta: float, short_factor, factor: Optional[float],
                         max_position_embeddings: int, original_max_position_embeddings: Optional[int] = None,
                         attention_factor: Optional[float] = None):
    """LongRoPE as the reference's Falcon runs it (src/transformers/modeling_rope_utils.py:242-302 called from
    modeling_falcon.py:128, once, without a length): every trained frequency divided by its entry of
    ``short_factor``; the table for long sequences (``long_factor``) is only ever taken by rotary modules that update
    "dynamic" types (modeling_falcon.py:155-157 asks for that word in the type's name), so it is never used.
    Returns (table, factor on cosines and sines): ``sqrt(1 + ln(factor) / ln(trained context))`` for a factor
    above 1 unless ``attention_factor`` is given; with ``original_max_position_embeddings`` the factor is the
    ratio of the two context lengths (:283-290)."""
    short = torch.as_tensor([float(v) for v in short_factor], dtype=torch.float32)
    if tuple(short.shape) != (head_dim // 2,):
        raise ValueError(f"short_factor needs {head_dim // 2} entries, got {tuple(short.shape)}")
    if original_max_position_embeddings:
        trained = int(original_max_position_embeddings)
        factor = max_position_embeddings / trained
    else:
        trained = int(max_position_embeddings)
    if attention_factor is None:
        if factor is None:
            raise ValueError("longrope needs a factor, an attention_factor or original_max_position_embeddings")
        attention_factor = 1.0 if factor <= 1.0 else math.sqrt(1 + math.log(factor) / math.log(trained))
    inv = 1.0 / (short * float(theta) ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    return inv, float(attention_factor)


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

    #: False: slopes, positions and their product are rounded to bfloat16 as the reference rounds them
    exact_bias = False

    def __init__(self, num_heads: int, bf16_compat: bool = True, scale: float = 1.0):
        """``bf16_compat=False`` leaves the reference's numbers for the exact ``slope * position`` in 32-bit
        (``alibi_bf16_compat: false`` in config.json); the default reproduces the reference.  ``scale``: what the
        bias is multiplied by when it joins the scores (the reference's Falcon: one over the root of the head size,
        :1081)."""
        self.num_heads = num_heads
        self.exact_bias = not bf16_compat
        self.scale = float(scale)
        slopes = alibi_slopes(num_heads)
        self.slopes = (slopes if self.exact_bias else slopes.bfloat16().float()).contiguous()

    def to(self, device) -> None:
        self.slopes = self.slopes.to(device)

    def score_bias(self) -> ScoreBias:
        return ScoreBias(self.slopes, "key", not self.exact_bias, self.scale)


register_part("positions", "none", NoPositions)
register_part("positions", "rotary", RotaryPositions)
register_part("positions", "alibi", AlibiPositions)
