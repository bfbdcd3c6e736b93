"""What a model *is*, as data: tensors, blocks, the order they run in, cache groups.

A builder registered for an architecture (``config.registry.register``) returns
a :class:`ModelSpec`.  Nothing in here knows Falcon; ``engine/falcon.py`` is the
one builder this package ships.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, List, Optional, Sequence, Tuple

# how a tensor is held on the device
MATRIX = "matrix"  # operand of a matrix product or a lookup table of activations: held in the compute dtype
VECTOR = "vector"  # norm weights, biases: always held in 32-bit (a 16-bit file value widens exactly)
INT = "int"  # integer tables: int32

# how random-weights mode fills a tensor (src/transformers/models/falcon/modeling_falcon.py:794-808)
INIT_NORMAL = "normal"  # N(0, std)
INIT_ONE_NOISE = "one_noise"  # 1 + N(0, noise)   (reference: ones)
INIT_ZERO_NOISE = "zero_noise"  # N(0, noise)     (reference: zeros)


@dataclasses.dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: Tuple[int, ...]
    kind: str = MATRIX
    init: str = INIT_NORMAL
    #: if the file lacks this tensor, use that other tensor's storage instead (tied output head)
    tied_to: Optional[str] = None
    #: A file may hold this tensor in pieces instead (a checkpoint with separate query, key and value matrices for
    #: a model that runs them as one): (name, shape) of each piece.  ``assemble`` makes the tensor of the pieces,
    #: given in this order (None: joined along the first dimension).  A file that holds the tensor under its own
    #: name is read as before; random weights are drawn and written whole.
    pieces: Tuple[Tuple[str, Tuple[int, ...]], ...] = ()
    assemble: Optional[Callable[[Sequence[Any]], Any]] = None


# kinds of per-sequence storage a group of layers can ask for
CACHE_FULL = "full"  # every key and value of the sequence
CACHE_WINDOW = "window"  # the last `window` keys and values
CACHE_STATE = "state"  # a tensor of fixed shape per sequence, zero at the sequence's start


@dataclasses.dataclass(frozen=True)
class CacheGroupSpec:
    """Storage that a set of layers with the same needs shares a page pool (or a state table) for."""

    name: str
    kind: str
    num_layers: int
    kv_heads: int = 0
    head_dim: int = 0
    window: Optional[int] = None
    state_shape: Tuple[int, ...] = ()
    state_dtype: Any = None  # None: 32-bit float


@dataclasses.dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: which block runs, and on which layer of which cache group.

    A block may appear in several entries (its weights are used twice), and two
    entries may name the same ``cache_layer``; an entry with ``write_cache=False``
    reads what another entry wrote in this step or earlier.
    """

    block: int
    cache_group: Optional[str] = None
    cache_layer: int = 0
    write_cache: bool = True


@dataclasses.dataclass
class ModelSpec:
    config: Any
    embedding: Any  # parts.Embedding
    blocks: List[Any]  # parts.Block
    order: List[LayerCall]
    final_norm: Any  # parts norm or None
    head: Any  # parts.OutputHead
    cache_groups: List[CacheGroupSpec]
    #: what the checkpoint's tensor names start with when the whole model was saved, and lack when only its body
    #: was (the reference's ``base_model_prefix`` plus a dot); "" if there is no such prefix
    base_prefix: str = ""
    #: False if a part reads the step's host-side lists (``ctx.slots`` ...) while it runs: such a step
    #: cannot be captured into a graph and replayed with other values
    supports_graphs: bool = True

    def parts(self) -> Sequence[Any]:
        out = [self.embedding, *self.blocks]
        if self.final_norm is not None:
            out.append(self.final_norm)
        out.append(self.head)
        return out

    def tensor_specs(self) -> List[TensorSpec]:
        """Every tensor the parts need; a part that appears twice (shared weights) counts once."""
        specs: List[TensorSpec] = []
        seen = {}
        for p in self.parts():
            for s in p.all_tensor_specs():
                if s.name in seen:
                    if seen[s.name] != s:
                        raise ValueError(f"tensor {s.name!r} is declared twice with different shapes or kinds")
                    continue
                seen[s.name] = s
                specs.append(s)
        return specs

    def check_sizes(self) -> None:
        """Every part's sizes against what the kernels take (``Part.check_sizes``): a configuration that cannot run
        is refused here, before a weight is read."""
        seen = set()
        for p in self.parts():
            if id(p) not in seen:
                seen.add(id(p))
                p.check_all_sizes()

    def validate(self) -> None:
        groups = {g.name: g for g in self.cache_groups}
        if len(groups) != len(self.cache_groups):
            raise ValueError("cache group names must be unique")
        written = set()
        for i, call in enumerate(self.order):
            if not (0 <= call.block < len(self.blocks)):
                raise ValueError(f"order[{i}] names block {call.block}, but there are {len(self.blocks)} blocks")
            if call.cache_group is None:
                continue
            g = groups.get(call.cache_group)
            if g is None:
                raise ValueError(f"order[{i}] names cache group {call.cache_group!r}, which is not declared")
            if not (0 <= call.cache_layer < g.num_layers):
                raise ValueError(f"order[{i}] names layer {call.cache_layer} of group {g.name!r} ({g.num_layers} layers)")
            key = (call.cache_group, call.cache_layer)
            if call.write_cache:
                if key in written and g.kind != CACHE_STATE:
                    raise ValueError(f"order[{i}]: cache layer {key} is written twice in one pass")
                written.add(key)
            elif key not in written:
                raise ValueError(f"order[{i}] reads cache layer {key} before any entry wrote it")
