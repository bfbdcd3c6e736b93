"""How norm, mixer and feed-forward stand in a block, and how the residual is summed.

The two arrangements of ``FalconDecoderLayer.forward``
(src/transformers/models/falcon/modeling_falcon.py:614-683):

parallel    ``x + (ffn(norm_ffn(x)) + mixer(norm_mixer(x)))``; with one norm both branches read
            the same normed input (:630-634, :648-676).  The sum is formed in that order:
            feed-forward plus mixer first (:673-674), then the residual (:676).
sequential  ``r = x + mixer(norm_in(x))``; ``r + ffn(norm_post(r))`` (:652-659, :676).

The additions ride in the last matrix product's epilogue of each branch, or, in steps of few tokens,
the products stay unreduced and the next norm forms the sum while it reads it (``ResidualSum``).
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .base import Part, ResidualSum, StepContext, register_part
from .linear import Linear, PendingProjection


def _can_defer(part: Part) -> bool:
    return bool(getattr(part, "can_defer", False))


def _normed(x, norm: Part, other: Optional[Part] = None):
    """``(x as a tensor, norm(x), other(x) or None)`` for a block input that may be a sum not formed yet."""
    if isinstance(x, ResidualSum):
        if hasattr(norm, "forward_sum"):
            return norm.forward_sum(x, other=other)
        x = x.tensor()
    if other is None:
        return x, norm.forward(x), None
    if hasattr(norm, "forward_pair"):  # two norms of one input in one pass, where the norm offers it
        a, m = norm.forward_pair(x, other)
    else:
        a, m = norm.forward(x), other.forward(x)
    return x, a, m


def _sum_parallel(ffn_out: PendingProjection, mixer_out: PendingProjection, x: torch.Tensor):
    """feed-forward + mixer + residual, in that order, formed now or left to the next norm."""
    both = PendingProjection.partial_pair(ffn_out, mixer_out)
    if both is not None:
        return ResidualSum([both[0], both[1], x])
    p = ffn_out.partial()
    if p is not None:
        return ResidualSum([p, mixer_out.partial() or mixer_out.run(), x])
    if ffn_out.additions_cost_a_pass():  # prompts: the next norm adds the three while it reads them
        return ResidualSum([ffn_out.run(), mixer_out.run(), x])
    return ffn_out.run(add1=mixer_out.run(), add2=x)


def _sum_sequential(out: PendingProjection, residual: torch.Tensor):
    p = out.partial()
    if p is not None:
        return ResidualSum([p, residual])
    if out.additions_cost_a_pass():
        return ResidualSum([out.run(), residual])
    return out.run(add1=residual)


class ParallelBlock(Part):
    accepts_sum = True

    def __init__(self, mixer: Part, feed_forward: Part, norm_mixer: Part, norm_ffn: Optional[Part] = None):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_mixer = norm_mixer
        self.norm_ffn = norm_ffn

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.norm_mixer, self.norm_ffn, self.mixer, self.feed_forward) if p is not None)

    def after_load(self) -> None:
        """With one norm both branches start from the same input: their first matrices are laid out side by
        side, so that prompts can run them as one product."""
        if self.norm_ffn is None and hasattr(self.mixer, "input_projection") and hasattr(self.feed_forward, "input_projection"):
            Linear.join(self.mixer.input_projection()[0], self.feed_forward.input_projection()[0])

    def forward(self, x, ctx: StepContext, call):
        x, a, m = _normed(x, self.norm_mixer, self.norm_ffn)
        if m is None:
            m = a
        kw_mixer, kw_ffn = {}, {}
        # both branches start with a product of the norm's output: one launch for the two in small steps
        if hasattr(self.mixer, "input_projection") and hasattr(self.feed_forward, "input_projection"):
            (lin_a, kw_a), (lin_m, kw_m) = self.mixer.input_projection(), self.feed_forward.input_projection()
            tail = self.mixer.projection_tail(ctx, call) if hasattr(self.mixer, "projection_tail") else None
            both = Linear.pair(lin_a, a, kw_a, lin_m, m, kw_m, tail=tail)
            if both is not None:
                kw_mixer["projected"], kw_ffn["projected"] = both
        if _can_defer(self.feed_forward) and _can_defer(self.mixer):
            # the branches' last products: one launch of partial sums where that pays, which the
            # next norm adds to the residual while it reads them
            out_a = self.mixer.forward(a, ctx, call, defer=True, **kw_mixer)
            out_m = self.feed_forward.forward(m, ctx, defer=True, **kw_ffn)
            return _sum_parallel(out_m, out_a, x)
        mixed = self.mixer.forward(a, ctx, call, **kw_mixer)
        return self.feed_forward.forward(m, ctx, add1=mixed, add2=x, **kw_ffn)


class SequentialBlock(Part):
    accepts_sum = True

    def __init__(self, mixer: Part, feed_forward: Part, norm_in: Part, norm_post: Part):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norm_in
        self.norm_post = norm_post

    def children(self) -> Sequence[Part]:
        return (self.norm_in, self.norm_post, self.mixer, self.feed_forward)

    def forward(self, x, ctx: StepContext, call):
        x, a, _ = _normed(x, self.norm_in)
        if _can_defer(self.mixer):
            r = _sum_sequential(self.mixer.forward(a, ctx, call, defer=True), x)
        else:
            r = self.mixer.forward(a, ctx, call, residual=x)
        r, m, _ = _normed(r, self.norm_post)
        if _can_defer(self.feed_forward):
            return _sum_sequential(self.feed_forward.forward(m, ctx, defer=True), r)
        return self.feed_forward.forward(m, ctx, add1=r)


register_part("block", "parallel", ParallelBlock)
register_part("block", "sequential", SequentialBlock)
