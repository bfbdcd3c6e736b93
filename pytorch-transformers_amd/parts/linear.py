"""Linear layers, the embedding table and the output head.

``y = x @ W.T``, then ``+ b`` as a second operation whose result is rounded to the
storage type, as the reference does on purpose
(src/transformers/models/falcon/modeling_falcon.py:64-72).  In 32-bit the whole
layer, with activation and residual additions, is one hand-written kernel with a
fixed summation order.  In bfloat16, steps of at most 128 tokens (decoding, short
prompts), and up to 256 where that was timed faster, run a hand-written kernel
that streams the weights once and applies bias, activation and additions in its
epilogue; larger steps use the vendor library's matrix
product (as the reference uses torch's), followed by one fused kernel for bias,
activation and additions.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..engine.spec import INIT_NORMAL, INIT_ZERO_NOISE, MATRIX, VECTOR, TensorSpec
from .base import PartialProduct, Part


class Linear(Part):
    def __init__(self, name: str, in_features: int, out_features: int, bias: bool, pieces=None, assemble=None):
        """``pieces``: (name, rows) of the matrices that a weight file may hold instead of this one (their ``.weight``
        and ``.bias`` under those names), which ``assemble`` (None: one after the other) makes into this one by
        their rows; the same function is applied to the biases."""
        self.name = name
        self.in_features = in_features
        self.out_features = out_features
        self.has_bias = bias
        self.pieces = tuple((str(n), int(rows)) for n, rows in (pieces or ()))
        self.assemble = assemble
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.name + ".weight", (self.out_features, self.in_features), MATRIX, INIT_NORMAL,
                            pieces=tuple((n + ".weight", (rows, self.in_features)) for n, rows in self.pieces),
                            assemble=self.assemble)]
        if self.has_bias:
            specs.append(TensorSpec(self.name + ".bias", (self.out_features,), VECTOR, INIT_ZERO_NOISE,
                                    pieces=tuple((n + ".bias", (rows,)) for n, rows in self.pieces),
                                    assemble=self.assemble))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name + ".weight"]
        self.bias = tensors[self.name + ".bias"] if self.has_bias else None
        self.joined = None  # (both matrices as one, the other Linear) after ``join``

    @staticmethod
    def join(first: "Linear", second: "Linear") -> bool:
        """Lay the two weight matrices out as one, ``first``'s rows then ``second``'s, if they are bfloat16 with
        one K: products of many rows with the same input can then run as one library product (``pair``).  The
        matrices themselves become views of the joined one, so nothing is held twice."""
        if first.joined is not None and first.joined[1] is second:
            return True
        a, b = first.weight, second.weight
        if not (a is not None and b is not None and a.dtype == b.dtype == torch.bfloat16 and a.is_cuda
                and a.device == b.device and a.dim() == b.dim() == 2 and a.shape[1] == b.shape[1]
                and a.shape[0] % 8 == 0 and b.shape[0] % 8 == 0):
            return False
        both = torch.empty((a.shape[0] + b.shape[0], a.shape[1]), dtype=a.dtype, device=a.device)
        both[:a.shape[0]].copy_(a)
        both[a.shape[0]:].copy_(b)
        first.weight, second.weight = both[:a.shape[0]], both[a.shape[0]:]
        first.joined = (both, second)
        return True

    def __call__(self, x: torch.Tensor, *, act: Optional[str] = None, add1=None, add2=None,
                 apply_bias: bool = True) -> torch.Tensor:
        """``act(x @ W.T + b) + add1 + add2``; with ``apply_bias=False`` the caller adds the bias itself."""
        bias = self.bias if apply_bias else None
        if x.dtype == torch.float32:
            return ops.gemm_f32(x, self.weight, bias, act, add1, add2)
        if ops.gemm_skinny_ok(x, self.weight):
            return ops.gemm_skinny_bf16(x, self.weight, bias, act, add1, add2)
        if ops.gemm_splitk_ok(x, self.weight):
            return ops.gemm_splitk_bf16(x, self.weight, bias, act, add1, add2)
        y = ops.library_mm_ksplit(x, self.weight, bias, act, add1, add2)
        if y is not None:
            return y
        y = ops.library_mm(x, self.weight)
        if bias is not None or act is not None or add1 is not None or add2 is not None:
            ops.epilogue_(y, bias, act, add1, add2)
        return y

    def with_tail(self, x: torch.Tensor, tail: "QkvTail") -> Optional["TailDone"]:
        """This product as a fused query_key_value projection whose launch also runs ``tail`` (a decode batch of
        17 rows and more, where the product is the split-K kernel's); else None, and the caller runs the two."""
        if not (ops.QKV_TAIL and x.dtype == torch.bfloat16 and tail.head_dim % 2 == 0
                and not ops.gemm_skinny_ok(x, self.weight) and ops.gemm_splitk_ok(x, self.weight)):
            return None
        return TailDone(ops.gemm_splitk_qkv(
            x, self.weight, tail.bias, tail.inv_freq, tail.cs_scale, tail.token_pos, tail.token_seq, tail.table,
            tail.k_pool, tail.v_pool, tail.num_heads, tail.kv_heads, tail.head_dim, tail.layout, tail.write_cache,
            **tail.how))

    @staticmethod
    def pair(first: "Linear", x1: torch.Tensor, kw1: dict, second: "Linear", x2: torch.Tensor, kw2: dict, tail=None):
        """``(first(x1, **kw1), second(x2, **kw2))`` from one matrix launch, in steps small enough for the
        decode kernels (same rows, no additions); else None.  ``tail`` (a ``QkvTail``) says what the caller will
        do with the first result; where the launch can do that itself, the first result comes back as
        ``TailDone(queries)``."""
        if not (x1.dtype == torch.bfloat16 and x1.shape[0] == x2.shape[0]):
            return None
        if any(k not in ("act", "apply_bias") for k in list(kw1) + list(kw2)):
            return None
        b1 = first.bias if kw1.get("apply_bias", True) else None
        b2 = second.bias if kw2.get("apply_bias", True) else None
        if (tail is not None and x1.shape == x2.shape and kw1.get("act") is None
                and ops.gemm_skinny_pair_qkv_ok(x1, first.weight, second.weight, tail.head_dim)):
            q, y2 = ops.gemm_skinny_pair_qkv(
                x1, first.weight, tail.bias, tail.inv_freq, tail.cs_scale, tail.token_pos, tail.token_seq, tail.table,
                tail.k_pool, tail.v_pool, tail.num_heads, tail.kv_heads, tail.head_dim, tail.layout, tail.write_cache,
                x2, second.weight, b2, kw2.get("act"), **tail.how)
            return TailDone(q), y2
        args = (x1, first.weight, x2, second.weight, b1, kw1.get("act"), b2, kw2.get("act"))
        if x1.shape == x2.shape and ops.gemm_skinny_ok(x1, first.weight) and ops.gemm_skinny_ok(x2, second.weight):
            return ops.gemm_skinny_pair_bf16(*args)
        if (x1 is x2 and x1.shape[0] > ops.SPLITK_MAX_ROWS and first.joined is not None and first.joined[1] is second
                and ops.joined_mm_pays(x1, first.joined[0], first.out_features)):
            # many rows, one input, the matrices side by side in memory: one library product where it was measured
            # faster than two; the results are blocks of columns of its output, each with its own epilogue
            y = ops.library_mm(x1, first.joined[0])
            y1, y2 = y[:, :first.out_features], y[:, first.out_features:]
            for yi, bias, act in ((y1, b1, kw1.get("act")), (y2, b2, kw2.get("act"))):
                if bias is not None or act is not None:
                    ops.epilogue_(yi, bias, act)
            return y1, y2
        # 17 rows and more: the pair launch where it beats the products on their own (``ops.pair_launch_pays``)
        if ops.pair_launch_pays(x1.shape[0], first.weight, second.weight) and \
                ops.gemm_splitk_pair_ok(x1, first.weight, x2, second.weight):
            if tail is not None and ops.QKV_TAIL and kw1.get("act") is None and tail.head_dim % 2 == 0:
                # the launch that adds the partial sums takes the fused rows to their end as well
                q, y2 = ops.gemm_splitk_pair_qkv(
                    x1, first.weight, tail.bias, tail.inv_freq, tail.cs_scale, tail.token_pos, tail.token_seq, tail.table,
                    tail.k_pool, tail.v_pool, tail.num_heads, tail.kv_heads, tail.head_dim, tail.layout, tail.write_cache,
                    x2, second.weight, b2, kw2.get("act"), **tail.how)
                return TailDone(q), y2
            return ops.gemm_splitk_pair_bf16(*args)
        return None

    def can_partial(self, x: torch.Tensor) -> bool:
        return x.dtype == torch.bfloat16 and ops.gemm_partial_ok(x, self.weight) and ops.layernorm_sum_ok(self.out_features)

    def partial(self, x: torch.Tensor) -> Optional[PartialProduct]:
        """The product left as partial sums for the next norm to add, where that pays; else None."""
        if self.can_partial(x):
            return PartialProduct(ops.gemm_splitk_partial(x, self.weight), self.bias)
        return None


class QkvTail:
    """What a mixer does with its fused query_key_value rows: bias, split into heads, rotation, queries out, keys
    and values into the cache pages.  ``run`` does it as a kernel of its own; a pair launch that is given the tail
    may do it in its epilogue instead (``Linear.pair``)."""

    def __init__(self, bias, rotation, token_pos, token_seq, table, k_pool, v_pool, num_heads: int,
                 kv_heads: int, head_dim: int, layout: str, write_cache: bool):
        """``rotation``: a ``positions.Rotation`` or None."""
        self.bias, self.rotation = bias, rotation
        self.inv_freq = None if rotation is None else rotation.inv_freq
        self.cs_scale = 1.0 if rotation is None else rotation.scale
        #: how the rotation lies in a head, as keywords of the launches that rotate
        self.how = {} if rotation is None else {"rotary_dim": rotation.rotary_dim, "pairing": rotation.pairing}
        self.token_pos, self.token_seq, self.table, self.k_pool, self.v_pool = token_pos, token_seq, table, k_pool, v_pool
        self.num_heads, self.kv_heads, self.head_dim, self.layout = num_heads, kv_heads, head_dim, layout
        self.write_cache = write_cache

    def run(self, fused: torch.Tensor) -> torch.Tensor:
        return ops.qkv_rope_cache(fused, self.bias, self.inv_freq, self.cs_scale, self.token_pos, self.token_seq,
                                  self.table, self.k_pool, self.v_pool, self.num_heads, self.kv_heads, self.head_dim,
                                  self.layout, write_cache=self.write_cache, **self.how)


class TailDone:
    """A first product whose tail the launch has already run: ``value`` is what the tail gives."""

    def __init__(self, value: torch.Tensor):
        self.value = value


class PendingProjection:
    """A part's last product, not run yet: the ``Linear`` and its input.  A mixer or feed-forward called
    with ``defer=True`` returns it, and the block chooses how to run it: on its own with the additions in
    its epilogue (``run``), left as partial sums for the next norm (``partial``), or together with the
    other branch's in one launch (``partial_pair``)."""

    def __init__(self, linear: Linear, x: torch.Tensor):
        self.linear, self.x = linear, x

    def run(self, add1=None, add2=None) -> torch.Tensor:
        return self.linear(self.x, add1=add1, add2=add2)

    def partial(self) -> Optional[PartialProduct]:
        return self.linear.partial(self.x)

    def additions_cost_a_pass(self) -> bool:
        """Whether tensors added to this product would be a pass of their own over the result: the vendor
        library's product of many rows, which has no epilogue of ours, with no bias to add.  The norm that reads
        the sum next can then form it while it reads (``ResidualSum``)."""
        x, lin = self.x, self.linear
        return (x.dtype == torch.bfloat16 and lin.bias is None and ops.layernorm_sum_ok(lin.out_features)
                and x.shape[0] >= ops.layernorm_sum_rows_min()
                and not ops.gemm_skinny_ok(x, lin.weight) and not ops.gemm_splitk_ok(x, lin.weight))

    @staticmethod
    def partial_pair(first: "PendingProjection", second: "PendingProjection"):
        """Both as partial sums from one launch, or None where that does not apply."""
        a, b = first, second
        if not (a.x.dtype == torch.bfloat16 and ops.layernorm_sum_ok(a.linear.out_features)
                and ops.gemm_partial_pair_ok(a.x, a.linear.weight, b.x, b.linear.weight)):
            return None
        pa, pb = ops.gemm_splitk_pair_partial(a.x, a.linear.weight, b.x, b.linear.weight)
        return PartialProduct(pa, a.linear.bias), PartialProduct(pb, b.linear.bias)


class Embedding(Part):
    """``h[t] = E[id_t]``, no scaling (src/transformers/models/falcon/modeling_falcon.py:835, :895-896)."""

    def __init__(self, name: str, vocab_size: int, hidden_size: int):
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.vocab_size, self.hidden_size), MATRIX, INIT_NORMAL)]

    def load(self, tensors) -> None:
        self.weight = tensors[self.name + ".weight"]

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.embed(self.weight, ids)


class OutputHead(Part):
    """``logits = h @ W.T`` in 32-bit, no bias; ``W`` is the embedding table when tied
    (src/transformers/models/falcon/modeling_falcon.py:1163-1168, :1230; the reference casts the
    rows it samples from to 32-bit, src/transformers/generation/utils.py:3247)."""

    def __init__(self, name: str, vocab_size: int, hidden_size: int, tied_to: Optional[str]):
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied_to = tied_to
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.vocab_size, self.hidden_size), MATRIX, INIT_NORMAL,
                           tied_to=self.tied_to)]

    def load(self, tensors) -> None:
        self.weight = tensors[self.name + ".weight"]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        if h.dtype == torch.float32:
            return ops.gemm_f32(h, self.weight)
        if ops.gemm_skinny_ok(h, self.weight):
            return ops.gemm_skinny_bf16(h, self.weight, out_f32=True)
        with ops.timed("library_mm", float(self.weight.numel()) * 2, 2.0 * h.shape[0] * self.weight.numel()):
            return torch.mm(h, self.weight.t(), out_dtype=torch.float32)
