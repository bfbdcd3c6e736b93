"""The cache: a slot per sequence, pages of a pool per layer group, and fixed-size state.

The reference's caches are per-layer tensors ``[batch, heads, length, head_dim]``
that grow by concatenation (``DynamicCache`` src/transformers/cache_utils.py:396-441)
or are allocated up front (``StaticCache`` :1134-1155, written with
``index_copy_`` :1183-1205); layers with different needs get tensors of
different shapes (``HybridCache`` :1626-1638) and fixed-size state lives in
``[layers, batch, ...]`` tables (``MambaCache`` :1813-1828).  A batch row is a
sequence's place for the whole call and its true length is implied by padding.

Here a sequence holds a *slot* (an integer) with an explicit length.  The bookkeeping (free lists,
page lists, lengths) lives in the host runtime (``csrc/host/runtime_host.cpp``); this class owns the
device tensors and is the runtime's Python face.  Each
layer group owns a pool of pages of ``page_size`` tokens; a slot's keys and
values are the pages its page list names, in order, so the position of a key is
its index in the slot.  Slots and pages go back to free lists when a sequence
ends and are handed out again; nothing is zeroed, because a slot's length says
what is valid.  Beyond the pages and slots that sequences can hold, every pool has one more page and every
state table one more row (``scratch_page``, ``scratch_slot``) that no sequence ever owns: rows that pad a
step to a fixed batch size (a captured decode step) write there, so that padding touches no sequence's
keys, values or state.  A group of kind ``window`` is laid out like a full one, but gives the pages that lie
wholly behind its window back to its pool as a sequence grows (their places in the page list hold
-1), so a long sequence holds about ``window / page_size`` pages of it.  Groups of kind ``state`` own a ``[max_slots, *shape]`` table per
layer that is zeroed when a slot is handed out.

The K pool has the layout ``[layer, page, kv_head, page_size, head_dim]``, the V pool
``[layer, page, kv_head, head_dim, page_size]``.
"""
from __future__ import annotations

import ctypes
from typing import Dict, List, Optional, Sequence

import torch

from .. import host
from ..engine.spec import CACHE_FULL, CACHE_STATE, CACHE_WINDOW, CacheGroupSpec

PAGE_SIZE = 64


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """The pool has too few free pages (or no free slot) for what a step needs."""


class _Group:
    """Storage of one layer group."""

    def __init__(self, spec: CacheGroupSpec, num_pages: int, max_slots: int, page_size: int, dtype, device):
        self.spec = spec
        self.page_size = page_size
        self.k = self.v = None
        self.state: Optional[torch.Tensor] = None
        self.paged = spec.kind in (CACHE_FULL, CACHE_WINDOW)
        self.window = int(spec.window or 0) if spec.kind == CACHE_WINDOW else 0
        self.index = -1  # among the paged groups, as the host runtime counts them
        if spec.kind == CACHE_WINDOW and self.window <= 0:
            raise CacheError(f"cache group {spec.name!r}: kind 'window' needs a positive window, got {spec.window!r}")
        if self.paged:
            # values are held transposed inside a page so that the attention kernels read eight
            # consecutive positions of one feature in one load
            # (one page more than sequences can hold: the scratch page of padding rows)
            self.k = torch.zeros((spec.num_layers, num_pages + 1, spec.kv_heads, page_size, spec.head_dim),
                                 dtype=dtype, device=device)
            self.v = torch.zeros((spec.num_layers, num_pages + 1, spec.kv_heads, spec.head_dim, page_size),
                                 dtype=dtype, device=device)
        elif spec.kind == CACHE_STATE:
            sd = spec.state_dtype or torch.float32
            # (one row more than there are slots: the scratch slot of padding rows)
            self.state = torch.zeros((spec.num_layers, max_slots + 1, *spec.state_shape), dtype=sd, device=device)
        else:
            raise CacheError(f"cache group {spec.name!r}: unknown kind {spec.kind!r}")


class PagedCache:
    """Slots, their lengths and page lists (kept by the host runtime), and the device storage of every group."""

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
        self._paged = [name for name, g in self.groups.items() if g.paged]
        for i, name in enumerate(self._paged):
            self.groups[name].index = i
        self._lib = host.load()
        self._h = self._lib.ptah_cache_new(self.max_slots, page_size, len(self._paged),
                                           host.int_array([self.num_pages] * len(self._paged)),
                                           host.int_array([self.groups[n].window for n in self._paged]))
        if not self._h:
            raise CacheError(host.last_error())

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.ptah_cache_delete(h)

    def _raise(self, rc: int):
        msg = host.last_error()
        for i, name in enumerate(self._paged):  # the runtime knows groups by number
            msg = msg.replace(f"group {i} ", f"group {name!r} ")
        raise (CacheFull if rc == host.ERR_FULL else CacheError)(msg)

    @property
    def scratch_slot(self) -> int:
        """A row of every state table that no sequence owns: where padding rows of a step keep their state."""
        return self.max_slots

    @property
    def scratch_page(self) -> int:
        """A page of every pool that no sequence owns: where padding rows of a step write keys and values."""
        return self.num_pages

    @property
    def handle(self):
        """The host runtime's handle of this cache (for ``plan_step``)."""
        return self._h

    # slots -------------------------------------------------------------
    def alloc(self) -> int:
        slot = self._lib.ptah_alloc(self._h)
        if slot < 0:
            self._raise(host.ERR_FULL)
        for g in self.groups.values():
            if g.state is not None:
                g.state[:, slot].zero_()
        return slot

    def free(self, slot: int) -> None:
        rc = self._lib.ptah_free(self._h, int(slot))
        if rc:
            self._raise(rc)

    def length(self, slot: int) -> int:
        n = self._lib.ptah_length(self._h, int(slot))
        if n < 0:
            self._raise(host.ERR_CACHE)
        return n

    def live_slots(self) -> List[int]:
        return [s for s in range(self.max_slots) if self._lib.ptah_is_live(self._h, s)]

    def free_pages(self, group: Optional[str] = None) -> int:
        names = [group] if group is not None else self._paged
        return min((self._lib.ptah_free_pages(self._h, self.groups[n].index) for n in names), default=self.num_pages)

    def free_slots(self) -> int:
        return self._lib.ptah_free_slots(self._h)

    # growth ------------------------------------------------------------
    def reserve(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """Give every slot the pages that ``new_tokens`` more tokens need; all or nothing."""
        rc = self._lib.ptah_reserve(self._h, len(slots), host.int_array([int(s) for s in slots]),
                                    host.int_array([int(n) for n in new_tokens]))
        if rc:
            self._raise(rc)

    def commit(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """The step has written ``new_tokens`` tokens of every slot."""
        rc = self._lib.ptah_commit(self._h, len(slots), host.int_array([int(s) for s in slots]),
                                   host.int_array([int(n) for n in new_tokens]))
        if rc:
            self._raise(rc)

    def page_list(self, group: str, slot: int) -> List[int]:
        gi = self.groups[group].index
        n = self._lib.ptah_page_count(self._h, gi, int(slot))
        if n < 0:
            self._raise(host.ERR_CACHE)
        out = (ctypes.c_int * max(1, n))()
        self._lib.ptah_pages(self._h, gi, int(slot), out)
        return list(out[:n])

    def paged_groups(self) -> List[str]:
        return list(self._paged)

    # storage -----------------------------------------------------------
    def kv_layer(self, group: str, layer: int):
        g = self.groups[group]
        return g.k[layer], g.v[layer]

    def state_layer(self, group: str, layer: int) -> torch.Tensor:
        return self.groups[group].state[layer]

    # fixed-size state: copies out and back -------------------------------------------------
    def snapshot_state(self, slot: int) -> Dict[str, torch.Tensor]:
        """A copy of everything of fixed size that ``slot`` holds, per state group ``[layers, *shape]`` (the
        reference clones its state tables when a sequence forks, src/transformers/cache_utils.py:1813-1847)."""
        if not self._lib.ptah_is_live(self._h, int(slot)):
            raise CacheError(f"slot {slot} is not allocated")
        return {name: g.state[:, int(slot)].clone() for name, g in self.groups.items() if g.state is not None}

    def restore_state(self, slot: int, snapshot: Dict[str, torch.Tensor]) -> None:
        """Put a ``snapshot_state`` back into ``slot`` (the same slot later, or another one that is to go on from
        that state)."""
        if not self._lib.ptah_is_live(self._h, int(slot)):
            raise CacheError(f"slot {slot} is not allocated")
        names = {name for name, g in self.groups.items() if g.state is not None}
        if set(snapshot) != names:
            raise CacheError(f"the snapshot holds the state groups {sorted(snapshot)}, this cache has {sorted(names)}")
        for name, t in snapshot.items():
            dst = self.groups[name].state[:, int(slot)]
            if tuple(t.shape) != tuple(dst.shape) or t.dtype != dst.dtype:
                raise CacheError(f"state group {name!r}: the snapshot is {tuple(t.shape)} {t.dtype}, the slot holds "
                                 f"{tuple(dst.shape)} {dst.dtype}")
            dst.copy_(t)

    def bytes_per_token(self) -> int:
        total = 0
        for g in self.groups.values():
            if g.k is not None:
                total += 2 * g.spec.num_layers * g.spec.kv_heads * g.spec.head_dim * g.k.element_size()
        return total

    def check_consistent(self) -> None:
        """Every page is either free or in exactly one live slot's list; used by tests and debug runs."""
        rc = self._lib.ptah_check(self._h)
        if rc:
            self._raise(rc)
