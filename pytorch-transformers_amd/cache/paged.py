"""The cache: a slot per sequence, pages of a pool per layer group, and fixed-size state.

The reference's caches are per-layer tensors ``[batch, heads, length, head_dim]``
that grow by concatenation (``DynamicCache`` src/transformers/cache_utils.py:396-441)
or are allocated up front (``StaticCache`` :1134-1155, written with
``index_copy_`` :1183-1205); layers with different needs get tensors of
different shapes (``HybridCache`` :1626-1638) and fixed-size state lives in
``[layers, batch, ...]`` tables (``MambaCache`` :1813-1828).  A batch row is a
sequence's place for the whole call and its true length is implied by padding.

Here a sequence holds a *slot* (an integer) with an explicit length.  Each
layer group owns a pool of pages of ``page_size`` tokens; a slot's keys and
values are the pages its page list names, in order, so the position of a key is
its index in the slot.  Slots and pages go back to free lists when a sequence
ends and are handed out again; nothing is zeroed, because a slot's length says
what is valid.  Groups of kind ``state`` own a ``[max_slots, *shape]`` table per
layer that is zeroed when a slot is handed out.

The K pool has the layout ``[layer, page, kv_head, page_size, head_dim]``, the V pool
``[layer, page, kv_head, head_dim, page_size]``.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..engine.spec import CACHE_FULL, CACHE_STATE, CACHE_WINDOW, CacheGroupSpec

PAGE_SIZE = 64


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """The pool has too few free pages (or no free slot) for what a step needs."""


class _FreeList:
    """Integers 0..n-1, handed out lowest first; returning one twice is an error."""

    def __init__(self, n: int, what: str):
        self.n = n
        self.what = what
        self._free = list(range(n - 1, -1, -1))  # pop() gives the lowest
        self._held = [False] * n

    def __len__(self):
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what} (all {self.n} are held)")
        i = self._free.pop()
        self._held[i] = True
        return i

    def give(self, i: int) -> None:
        if not (0 <= i < self.n):
            raise CacheError(f"{self.what} {i} does not exist (0..{self.n - 1})")
        if not self._held[i]:
            raise CacheError(f"{self.what} {i} is freed twice (or was never handed out)")
        self._held[i] = False
        self._free.append(i)
        # keep "lowest first" so that reuse is immediate and deterministic
        self._free.sort(reverse=True)

    def held(self, i: int) -> bool:
        return 0 <= i < self.n and self._held[i]

    def held_count(self) -> int:
        return self.n - len(self._free)


class _Group:
    """Storage of one layer group."""

    def __init__(self, spec: CacheGroupSpec, num_pages: int, max_slots: int, page_size: int, dtype, device):
        self.spec = spec
        self.page_size = page_size
        self.k = self.v = None
        self.state: Optional[torch.Tensor] = None
        self.pages: Optional[_FreeList] = None
        if spec.kind == CACHE_FULL:
            # values are held transposed inside a page so that the attention kernels read eight
            # consecutive positions of one feature in one load
            self.k = torch.zeros((spec.num_layers, num_pages, spec.kv_heads, page_size, spec.head_dim),
                                 dtype=dtype, device=device)
            self.v = torch.zeros((spec.num_layers, num_pages, spec.kv_heads, spec.head_dim, page_size),
                                 dtype=dtype, device=device)
            self.pages = _FreeList(num_pages, f"page of cache group {spec.name!r}")
        elif spec.kind == CACHE_STATE:
            sd = spec.state_dtype or torch.float32
            self.state = torch.zeros((spec.num_layers, max_slots, *spec.state_shape), dtype=sd, device=device)
        elif spec.kind == CACHE_WINDOW:
            raise CacheError(
                f"cache group {spec.name!r}: kind 'window' is declared in the interface but no kernel reads a "
                "ring of pages yet; use 'full'")
        else:
            raise CacheError(f"cache group {spec.name!r}: unknown kind {spec.kind!r}")

    def pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size if self.pages is not None else 0


class PagedCache:
    """Slots, their lengths and page lists, and the device storage of every group."""

    def __init__(self, groups: Sequence[CacheGroupSpec], max_tokens: int, dtype: torch.dtype, device,
                 *, max_slots: Optional[int] = None, page_size: int = PAGE_SIZE):
        if max_tokens <= 0:
            raise CacheError("max_tokens must be positive")
        self.page_size = page_size
        self.num_pages = (max_tokens + page_size - 1) // page_size
        # every live sequence holds at least one page, so more slots than pages are never needed
        self.max_slots = int(max_slots) if max_slots is not None else self.num_pages
        self.dtype = dtype
        self.device = torch.device(device)
        self.groups: Dict[str, _Group] = {
            g.name: _Group(g, self.num_pages, self.max_slots, page_size, dtype, self.device) for g in groups}
        self._slots = _FreeList(self.max_slots, "slot")
        self._length: List[int] = [0] * self.max_slots
        self._pages: Dict[str, List[List[int]]] = {
            name: [[] for _ in range(self.max_slots)] for name, g in self.groups.items() if g.pages is not None}

    # slots -------------------------------------------------------------
    def alloc(self) -> int:
        slot = self._slots.take()
        self._length[slot] = 0
        for g in self.groups.values():
            if g.state is not None:
                g.state[:, slot].zero_()
        return slot

    def free(self, slot: int) -> None:
        self._check(slot)
        for name, table in self._pages.items():
            pool = self.groups[name].pages
            for p in table[slot]:
                pool.give(p)
            table[slot] = []
        self._length[slot] = 0
        self._slots.give(slot)

    def _check(self, slot: int) -> None:
        if not self._slots.held(slot):
            raise CacheError(f"slot {slot} is not allocated")

    def length(self, slot: int) -> int:
        self._check(slot)
        return self._length[slot]

    def live_slots(self) -> List[int]:
        return [s for s in range(self.max_slots) if self._slots.held(s)]

    def free_pages(self, group: Optional[str] = None) -> int:
        names = [group] if group is not None else list(self._pages)
        return min((len(self.groups[n].pages) for n in names), default=self.num_pages)

    def free_slots(self) -> int:
        return len(self._slots)

    # growth ------------------------------------------------------------
    def reserve(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """Give every slot the pages that ``new_tokens`` more tokens need; all or nothing."""
        if len(set(slots)) != len(slots):
            raise CacheError(f"a slot appears twice in one step: {list(slots)}")
        for s in slots:
            self._check(s)
        for name, table in self._pages.items():
            g = self.groups[name]
            need = 0
            for s, n in zip(slots, new_tokens):
                need += max(0, g.pages_for(self._length[s] + n) - len(table[s]))
            if need > len(g.pages):
                raise CacheFull(
                    f"cache group {name!r} needs {need} more pages of {self.page_size} tokens for this step, "
                    f"{len(g.pages)} of {g.pages.n} are free")
        for name, table in self._pages.items():
            g = self.groups[name]
            for s, n in zip(slots, new_tokens):
                while len(table[s]) < g.pages_for(self._length[s] + n):
                    table[s].append(g.pages.take())

    def commit(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """The step has written ``new_tokens`` tokens of every slot."""
        for s, n in zip(slots, new_tokens):
            self._length[s] += n

    def page_list(self, group: str, slot: int) -> List[int]:
        self._check(slot)
        return self._pages[group][slot]

    def paged_groups(self) -> List[str]:
        return list(self._pages)

    # storage -----------------------------------------------------------
    def kv_layer(self, group: str, layer: int):
        g = self.groups[group]
        return g.k[layer], g.v[layer]

    def state_layer(self, group: str, layer: int) -> torch.Tensor:
        return self.groups[group].state[layer]

    def bytes_per_token(self) -> int:
        total = 0
        for g in self.groups.values():
            if g.k is not None:
                total += 2 * g.spec.num_layers * g.spec.kv_heads * g.spec.head_dim * g.k.element_size()
        return total

    def check_consistent(self) -> None:
        """Every page is either free or in exactly one live slot's list; used by tests and debug runs."""
        for name, table in self._pages.items():
            g = self.groups[name]
            seen = {}
            for s in range(self.max_slots):
                if table[s] and not self._slots.held(s):
                    raise CacheError(f"freed slot {s} still lists pages {table[s]} in group {name!r}")
                if self._slots.held(s) and len(table[s]) < g.pages_for(self._length[s]):
                    raise CacheError(f"slot {s} has length {self._length[s]} but only {len(table[s])} pages")
                for p in table[s]:
                    if p in seen:
                        raise CacheError(f"page {p} of group {name!r} is held by slots {seen[p]} and {s}")
                    if not g.pages.held(p):
                        raise CacheError(f"page {p} of group {name!r} is in slot {s}'s list and in the free list")
                    seen[p] = s
            if len(seen) != g.pages.held_count():
                raise CacheError(
                    f"group {name!r}: {g.pages.held_count()} pages are marked held, {len(seen)} are in slot lists")
