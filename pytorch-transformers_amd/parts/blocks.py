"""How norm, mixer and feed-forward stand in a block, and how the residual is summed.

The two arrangements of ``FalconDecoderLayer.forward``
(src/transformers/models/falcon/modeling_falcon.py:614-683):

parallel    ``x + (ffn(norm_ffn(x)) + mixer(norm_mixer(x)))``; with one norm both branches read
            the same normed input (:630-634, :648-676).  The sum is formed in that order:
            feed-forward plus mixer first (:673-674), then the residual (:676).
sequential  ``r = x + mixer(norm_in(x))``; ``r + ffn(norm_post(r))`` (:652-659, :676).

The additions ride in the last matrix product's epilogue of each branch.  In the parallel block the
feed-forward's first product does not depend on the mixer, so it may run beside it on a second stream.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .base import Part, StepContext, register_part


class ParallelBlock(Part):
    def __init__(self, mixer: Part, feed_forward: Part, norm_mixer: Part, norm_ffn: Optional[Part] = None):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_mixer = norm_mixer
        self.norm_ffn = norm_ffn

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.norm_mixer, self.norm_ffn, self.mixer, self.feed_forward) if p is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, call) -> torch.Tensor:
        if self.norm_ffn is None:
            a = m = self.norm_mixer.forward(x)
        else:
            a, m = self.norm_mixer.forward_pair(x, self.norm_ffn)
        side = ctx.side_stream
        if side is None or not hasattr(self.feed_forward, "forward_up"):
            mixed = self.mixer.forward(a, ctx, call)
            return self.feed_forward.forward(m, ctx, add1=mixed, add2=x)
        # The feed-forward's first product needs only the norm, not the mixer: it runs on a second
        # stream beside projection, rotation, attention and output projection, and the two meet at the
        # feed-forward's second product, whose epilogue sums the branches and the residual.
        main = torch.cuda.current_stream()
        side.wait_stream(main)
        with torch.cuda.stream(side):
            h = self.feed_forward.forward_up(m, ctx)
        mixed = self.mixer.forward(a, ctx, call)
        main.wait_stream(side)
        return self.feed_forward.forward_down(h, ctx, add1=mixed, add2=x)


class SequentialBlock(Part):
    def __init__(self, mixer: Part, feed_forward: Part, norm_in: Part, norm_post: Part):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norm_in
        self.norm_post = norm_post

    def children(self) -> Sequence[Part]:
        return (self.norm_in, self.norm_post, self.mixer, self.feed_forward)

    def forward(self, x: torch.Tensor, ctx: StepContext, call) -> torch.Tensor:
        r = self.mixer.forward(self.norm_in.forward(x), ctx, call, residual=x)
        return self.feed_forward.forward(self.norm_post.forward(r), ctx, add1=r)


register_part("block", "parallel", ParallelBlock)
register_part("block", "sequential", SequentialBlock)
