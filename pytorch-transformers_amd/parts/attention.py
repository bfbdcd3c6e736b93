"""Attention as a token mixer: fused projection, heads, positions, cache, scores, output projection.

Follows ``FalconAttention.forward``
(src/transformers/models/falcon/modeling_falcon.py:326-458) on its default
branch (``scaled_dot_product_attention``, :371-386 and :407-422), with these
differences of layout, none of value: tokens of all sequences lie end to end
instead of in a padded batch; keys and values are kept once per KV head (the
reference broadcasts them to every query head before caching, :286-289); the
causal mask is implied by each token's position instead of being a tensor.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

from .. import ops
from .base import Part, StepContext, register_part
from .linear import Linear, PendingProjection, QkvTail, TailDone
from .positions import as_rotation, as_score_bias


def fused_rows(num_heads: int, kv_heads: int, head_dim: int, qkv_layout: str):
    """A function that lays the rows of separate query, key and value projections (heads in order) out as the fused
    projection's in ``qkv_layout`` (the row orders of src/transformers/models/falcon/modeling_falcon.py:264-294):
    ``grouped``: per KV head its query heads, its key, its value; ``tail``: all query heads, the key, the value
    (one KV head); ``interleaved``: per head query, key, value (as many KV heads as heads).  All three are the
    grouped order at their head counts."""
    if (qkv_layout == "tail" and kv_heads != 1) or (qkv_layout == "interleaved" and kv_heads != num_heads):
        raise ValueError(f"the {qkv_layout} layout does not go with {num_heads} heads and {kv_heads} kv heads")

    def assemble(parts):
        q, k, v = parts
        rest = tuple(q.shape[1:])
        per = [t.reshape(kv_heads, -1, *rest) for t in (q, k, v)]  # [kv head, its rows, ...]
        return torch.cat(per, dim=1).reshape(-1, *rest)

    return assemble


class AttentionMixer(Part):
    def __init__(self, name: str, hidden_size: int, num_heads: int, kv_heads: int, head_dim: int, qkv_layout: str,
                 bias: bool, positions: Part, qkv_name: str = "query_key_value", out_name: str = "dense",
                 window: int = 0, qkv_pieces: Optional[Sequence[str]] = None):
        """``qkv_pieces``: the names of separate query, key and value projections (``("q_proj", "k_proj", "v_proj")``)
        that a weight file may hold in place of the fused one; their rows, heads in order, are laid out in
        ``qkv_layout`` when the weights are read, and the model runs the fused product either way."""
        if num_heads % kv_heads:
            raise ValueError(f"heads ({num_heads}) must be a multiple of kv heads ({kv_heads})")
        if qkv_layout not in ops.QKV_LAYOUT_CODES:
            raise ValueError(f"unknown qkv layout {qkv_layout!r}")
        self.name = name
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.kv_heads = kv_heads
        self.head_dim = head_dim
        self.qkv_layout = qkv_layout
        self.positions = positions
        #: 0, or how many of the last positions a token attends to (itself included); its cache group is then
        #: of kind ``window`` with the same number, and gives back the pages that fall behind
        self.window = int(window)
        self.scale = 1.0 / math.sqrt(head_dim)  # modeling_falcon.py:250
        pieces = assemble = None
        if qkv_pieces is not None:
            if len(qkv_pieces) != 3:
                raise ValueError(f"{name}: qkv_pieces names the query, key and value projections, got {qkv_pieces!r}")
            pieces = [(f"{name}.{n}", rows * head_dim) for n, rows in zip(qkv_pieces, (num_heads, kv_heads, kv_heads))]
            assemble = fused_rows(num_heads, kv_heads, head_dim, qkv_layout)
        self.qkv = Linear(f"{name}.{qkv_name}", hidden_size, (num_heads + 2 * kv_heads) * head_dim, bias, pieces, assemble)
        self.out = Linear(f"{name}.{out_name}", num_heads * head_dim, hidden_size, bias)

    def children(self) -> Sequence[Part]:
        return (self.qkv, self.out, self.positions)

    can_defer = True

    def check_sizes(self) -> None:
        rot = as_rotation(self.positions.rotation())
        problem = ops.attention_sizes_problem(self.num_heads, self.kv_heads, self.head_dim,
                                              rot is not None or hasattr(self.positions, "rotation_for"))
        if problem is None and rot is not None:
            problem = ops.rotation_problem(self.head_dim, rot.rotary_dim, rot.pairing)
        bias = as_score_bias(self.positions.score_bias(), self.head_dim)
        if problem is None and bias is not None:
            problem = ops.score_bias_problem(bias.of, bias.bf16)
        if problem is not None:
            raise ValueError(f"{self.name}: {problem}")

    def input_projection(self):
        """The first product of ``forward`` and how it is called: a block may run it together with another
        part's and hand the result back as ``projected``."""
        return self.qkv, {"apply_bias": False}

    def projection_tail(self, ctx: StepContext, call) -> QkvTail:
        """What ``forward`` does with the first product's rows; a block that runs that product in a launch of its
        own may hand this to the launch (``Linear.pair``)."""
        k_pool, v_pool = ctx.cache.kv_layer(call.cache_group, call.cache_layer)
        # a position encoding whose rotation depends on the step (frequencies per sequence) offers rotation_for
        rot = as_rotation(self.positions.rotation_for(ctx) if hasattr(self.positions, "rotation_for")
                          else self.positions.rotation())
        return QkvTail(self.qkv.bias, rot, ctx.token_pos, ctx.token_seq, ctx.block_tables[call.cache_group],
                       k_pool, v_pool, self.num_heads, self.kv_heads, self.head_dim, self.qkv_layout, call.write_cache)

    def forward(self, x: torch.Tensor, ctx: StepContext, call, residual: Optional[torch.Tensor] = None,
                defer: bool = False, projected=None):
        """Attention of the step's tokens over the cache, projected out, plus ``residual``.  With ``defer``
        the output projection comes back not run (``PendingProjection``); the caller adds the residual.
        ``projected``: the first product, run by the caller, or ``TailDone(queries)`` if its launch has also
        rotated it and written the cache."""
        k_pool, v_pool = ctx.cache.kv_layer(call.cache_group, call.cache_layer)
        table = ctx.block_tables[call.cache_group]
        if projected is None:
            projected = self.qkv.with_tail(x, self.projection_tail(ctx, call))
        if isinstance(projected, TailDone):
            q = projected.value
        else:
            fused = projected if projected is not None else self.qkv(x, apply_bias=False)
            q = self.projection_tail(ctx, call).run(fused)
        bias = as_score_bias(self.positions.score_bias(), self.head_dim)
        if bias is None:
            o = ops.attention(q, k_pool, v_pool, table, ctx, None, self.scale, self.window)
        else:
            o = ops.attention(q, k_pool, v_pool, table, ctx, bias.slopes, self.scale, self.window,
                              alibi_exact=not bias.bf16, bias_of=bias.of, bias_scale=bias.scale)
        if defer:
            return PendingProjection(self.out, o)
        return self.out(o, add1=residual)


register_part("mixer", "attention", AttentionMixer)
