"""Planning a step on the host: from (slot, tokens, wanted places) per sequence to flat integer arrays.

The reference feeds a padded ``[batch, T]`` matrix with an attention mask and derives positions from
the mask (src/transformers/generation/utils.py:349-481; ``position_ids`` :409-416).  Here the
tokens of all sequences lie end to end without padding and a token's position is its sequence's
cached length plus its index in the step, which is what the mask arithmetic yields for left-padded
rows.  All arrays go to the device in one int32 buffer.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import Dict, List, Optional, Sequence, Union

import numpy as np

Want = Union[str, Sequence[Sequence[int]], None]


class StepError(ValueError):
    pass


@dataclasses.dataclass
class StepPlan:
    slots: List[int]
    new_tokens: List[int]  # tokens each sequence brings
    starts: List[int]  # cached length of each sequence before the step
    token_ids: np.ndarray  # [M]
    token_seq: np.ndarray  # [M]
    token_pos: np.ndarray  # [M]
    cu_tokens: np.ndarray  # [n + 1]
    logit_rows: np.ndarray  # [R] indices into the M tokens
    rows_per_seq: List[int]
    block_tables: Dict[str, np.ndarray]  # group -> [n, pages]
    #: all of the arrays above in one int32 buffer, in the order token_ids, token_seq, token_pos, cu_tokens,
    #: starts, slots, logit_rows, then one page table per group; ``sizes`` are the pieces' lengths
    buffer: Optional[np.ndarray] = None
    sizes: Optional[List[int]] = None

    @property
    def n_seqs(self) -> int:
        return len(self.slots)

    @property
    def n_tokens(self) -> int:
        return int(self.token_ids.shape[0])

    @property
    def is_decode(self) -> bool:
        return all(n == 1 for n in self.new_tokens)

    @property
    def max_len(self) -> int:
        return max(s + n for s, n in zip(self.starts, self.new_tokens))

    @property
    def total_len(self) -> int:
        return sum(s + n for s, n in zip(self.starts, self.new_tokens))


_WANT_MODES = {"none": 0, "last": 1, "all": 2}


def plan_step(cache, slots: Sequence[int], tokens: Sequence[Sequence[int]], want: Want, vocab_size: int) -> StepPlan:
    """Check a step's arguments, reserve cache pages for it and lay its arrays out (in the host runtime)."""
    from .. import host
    from ..cache.paged import CacheError, CacheFull

    slots = [int(s) for s in slots]
    if len(slots) == 0:
        raise StepError("a step needs at least one sequence")
    if len(tokens) != len(slots):
        raise StepError(f"{len(slots)} slots but {len(tokens)} token lists")
    n = len(slots)
    new_tokens = [len(t) for t in tokens]
    flat = np.ascontiguousarray(np.concatenate([np.asarray(t, dtype=np.int64).reshape(-1) for t in tokens])
                                if sum(new_tokens) else np.zeros(0, dtype=np.int64))
    counts = places = None
    if want is None or isinstance(want, str):
        key = "none" if want is None else want
        if key not in _WANT_MODES:
            raise StepError(f"want must be 'last', 'all', 'none' or a list of places per sequence, got {want!r}")
        mode = _WANT_MODES[key]
    else:
        want = [[int(p) for p in w] for w in want]
        if len(want) != n:
            raise StepError(f"want has {len(want)} entries for {n} sequences")
        mode = 3
        counts = host.int_array([len(w) for w in want])
        places = host.int_array([p for w in want for p in w])
    lib = host.load()
    sizes = (ctypes.c_int * (7 + len(cache.paged_groups())))()
    rc = lib.ptah_plan_step(cache.handle, n, host.int_array(slots), host.int_array(new_tokens),
                            flat.ctypes.data_as(ctypes.POINTER(ctypes.c_longlong)), int(vocab_size), mode, counts,
                            places, sizes)
    if rc:
        msg = host.last_error()
        raise {host.ERR_STEP: StepError, host.ERR_FULL: CacheFull}.get(rc, CacheError)(msg)
    sizes = list(sizes)
    total = sum(sizes)
    buf = np.ctypeslib.as_array(lib.ptah_plan_data(cache.handle), shape=(total,)).copy()  # the runtime reuses its buffer
    views = np.split(buf, np.cumsum(sizes)[:-1])
    M, R = sizes[0], sizes[6]
    rows = views[6]
    if mode == 3:
        rows_per_seq = [len(w) for w in want]
    else:
        rows_per_seq = [0] * n if mode == 0 else [1] * n if mode == 1 else list(new_tokens)
    tables = {g: views[7 + i].reshape(n, -1) for i, g in enumerate(cache.paged_groups())}
    return StepPlan(slots=slots, new_tokens=new_tokens, starts=views[4].tolist(), token_ids=views[0], token_seq=views[1],
                    token_pos=views[2], cu_tokens=views[3], logit_rows=rows, rows_per_seq=rows_per_seq,
                    block_tables=tables, buffer=buf, sizes=sizes)
