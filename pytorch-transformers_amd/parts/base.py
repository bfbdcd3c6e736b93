"""Interfaces of the parts a model is put together from, and the table of part kinds.

A part is built from sizes and constants only; it never sees a model
configuration and does not know which model it is in.  Every part

* lists the tensors it needs (``tensor_specs``) under the names the weight file
  uses, and takes them from a dict by those names (``load``);
* works on activations ``[tokens, features]`` of all sequences of a step laid
  end to end; which token belongs to which sequence, and where it stands, is in
  the :class:`StepContext`.

Kinds and their ``forward``:

=============  ==================================================================
mixer          ``forward(x, ctx, call, residual=None) -> [tokens, hidden]``; reads
               and writes the cache layer that ``call`` names (keys and values, or
               a state table); ``residual`` is added to the result if given
feed_forward   ``forward(x, ctx, add1=None, add2=None) -> [tokens, hidden]``
norm           ``forward(x, rows=None) -> [tokens, hidden]`` (``rows``: int32
               indices of the rows to take); ``forward_pair(x, other)`` may fuse
               two norms of the same input
positions      ``rotation() -> (inv_freq or None, scale)`` for queries and keys,
               ``score_bias() -> per-head slopes or None`` for attention scores;
               optionally ``rotation_for(ctx) -> (table, scale)`` where the table may
               have a row per sequence of the step (frequencies that follow a length)
block          ``forward(x, ctx, call) -> x``: the arrangement of the above
=============  ==================================================================

Optional: a mixer or feed-forward that sets ``can_defer = True`` and is called with
``defer=True`` returns its last product not run, as a ``PendingProjection`` (the
``Linear`` and its input; residual and additions are then the caller's), and one
with ``input_projection()`` lets the block run its first product and hand the result
in as ``projected``.  A block may so run two branches' products in one launch, and
leave the last ones as 32-bit partial sums (:class:`PartialProduct`) in a
:class:`ResidualSum` that it returns in place of a tensor.  A norm with
``forward_sum(sum, rows=None, other=None, want_x=True) -> (x, normed, normed_other)``
forms such a sum while it normalises it; a block with ``accepts_sum = True`` takes one
as its input.  Everything else receives plain tensors.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Sequence

import torch

from ..engine.spec import TensorSpec

_KINDS = ("mixer", "feed_forward", "norm", "positions", "block")
_TABLE: Dict[str, Dict[str, type]] = {k: {} for k in _KINDS}


def register_part(kind: str, name: str, cls: type, *, exist_ok: bool = False) -> type:
    if kind not in _TABLE:
        raise ValueError(f"unknown part kind {kind!r}; kinds: {_KINDS}")
    if not exist_ok and name in _TABLE[kind]:
        raise ValueError(f"{kind} {name!r} is already registered")
    _TABLE[kind][name] = cls
    return cls


def make_part(kind: str, name: str, **params):
    try:
        cls = _TABLE[kind][name]
    except KeyError:
        raise ValueError(f"no {kind} named {name!r}; registered: {sorted(_TABLE.get(kind, {}))}") from None
    return cls(**params)


def registered_parts(kind: str) -> List[str]:
    return sorted(_TABLE[kind])


class Part:
    """Base of all parts: tensors by name."""

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take this part's tensors out of ``tensors`` (already on the device, in device types)."""

    def children(self) -> Sequence["Part"]:
        return ()

    def all_tensor_specs(self) -> List[TensorSpec]:
        out = list(self.tensor_specs())
        for c in self.children():
            out.extend(c.all_tensor_specs())
        return out

    def load_all(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.load(tensors)
        for c in self.children():
            c.load_all(tensors)

    def check_sizes(self) -> None:
        """Raise ``ValueError`` if no kernel takes this part's sizes; called before a weight is read or drawn."""

    def check_all_sizes(self) -> None:
        self.check_sizes()
        for c in self.children():
            c.check_all_sizes()


@dataclasses.dataclass
class PartialProduct:
    """A matrix product that its kernel left as 32-bit partial sums over ranges of K, ``[ranges, tokens,
    features]``, with the bias still to be added.  Whoever reads it adds the ranges in order, rounds, and adds
    the bias: the value the product's own epilogue would have stored."""

    parts: torch.Tensor
    bias: Optional[torch.Tensor] = None

    def term(self):
        return (self.parts, self.bias)


class ResidualSum:
    """The residual stream as a sum that is not formed yet: products first, then tensors, added in that
    order and rounded once.  A block may return it in place of a tensor; the norm that reads it next forms
    the sum in the same pass (``forward_sum``), and ``tensor()`` forms it for anyone else."""

    def __init__(self, terms: Sequence[Any]):
        self.terms = [t for t in terms if t is not None]
        first = self.terms[0]
        self.features = (first.parts if isinstance(first, PartialProduct) else first).shape[-1]

    def kernel_terms(self):
        return [t.term() if isinstance(t, PartialProduct) else t for t in self.terms]

    def tensor(self) -> torch.Tensor:
        from .. import ops

        if len(self.terms) == 1 and not isinstance(self.terms[0], PartialProduct):
            return self.terms[0]
        return ops.layernorm_sum(self.kernel_terms(), self.features)[0]


def as_tensor(x):
    """A tensor from what a part may hand on: a tensor, a ``PartialProduct`` or a ``ResidualSum``."""
    if isinstance(x, PartialProduct):
        return ResidualSum([x]).tensor()
    if isinstance(x, ResidualSum):
        return x.tensor()
    return x


@dataclasses.dataclass
class StepContext:
    """What one step's tokens are: built once per step by the engine, read by every part."""

    dtype: torch.dtype
    device: torch.device
    n_seqs: int
    n_tokens: int
    #: per token: index of its sequence in this step, and its position in that sequence
    token_seq: torch.Tensor
    token_pos: torch.Tensor
    #: per sequence: first token's offset in the step (n_seqs + 1 entries), cached length before the step
    cu_tokens: torch.Tensor
    seq_start: torch.Tensor
    #: per sequence: its slot (row of state tables)
    seq_slot: torch.Tensor
    #: per paged cache group: [n_seqs, pages] page ids
    block_tables: Dict[str, torch.Tensor]
    cache: Any
    #: host copies, for launch geometry
    slots: List[int]
    new_tokens: List[int]
    starts: List[int]
    #: True if every sequence brings exactly one token
    is_decode: bool = False
    #: upper bound of any sequence's length after this step, used to size launches
    max_len: int = 0
    #: upper bound of the sequences' mean length after this step (0: not known, take ``max_len``); launches
    #: may be shaped by it, but no result depends on it
    mean_len: int = 0
    extras: Dict[str, Any] = dataclasses.field(default_factory=dict)
