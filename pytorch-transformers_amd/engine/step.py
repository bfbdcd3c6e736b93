"""Planning a step on the host: from (slot, tokens, wanted places) per sequence to flat integer arrays.

The reference feeds a padded ``[batch, T]`` matrix with an attention mask and derives positions from
the mask (src/transformers/generation/utils.py:349-481; ``position_ids`` :409-416).  Here the
tokens of all sequences lie end to end without padding and a token's position is its sequence's
cached length plus its index in the step, which is what the mask arithmetic yields for left-padded
rows.  All arrays go to the device in one int32 buffer.
"""
from __future__ import annotations

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


def normalize_want(want: Want, new_tokens: Sequence[int]) -> List[List[int]]:
    """``"last"``, ``"all"``, ``None`` (nothing) or explicit places per sequence -> lists of places."""
    if want is None or want == "none":
        return [[] for _ in new_tokens]
    if want == "last":
        return [[n - 1] for n in new_tokens]
    if want == "all":
        return [list(range(n)) for n in new_tokens]
    if isinstance(want, str):
        raise StepError(f"want must be 'last', 'all', 'none' or a list of places per sequence, got {want!r}")
    want = [list(w) for w in want]
    if len(want) != len(new_tokens):
        raise StepError(f"want has {len(want)} entries for {len(new_tokens)} sequences")
    for i, (w, n) in enumerate(zip(want, new_tokens)):
        for p in w:
            if not (0 <= int(p) < n):
                raise StepError(f"sequence {i} wants the logits at place {p}, but brings {n} tokens")
    return want


def plan_step(cache, slots: Sequence[int], tokens: Sequence[Sequence[int]], want: Want, vocab_size: int) -> StepPlan:
    """Check a step's arguments, reserve cache pages for it and lay its arrays out."""
    slots = [int(s) for s in slots]
    if len(slots) == 0:
        raise StepError("a step needs at least one sequence")
    if len(tokens) != len(slots):
        raise StepError(f"{len(slots)} slots but {len(tokens)} token lists")
    new_tokens = [len(t) for t in tokens]
    for i, n in enumerate(new_tokens):
        if n == 0:
            raise StepError(f"sequence {i} (slot {slots[i]}) brings no tokens")
    flat = np.concatenate([np.asarray(t, dtype=np.int64).reshape(-1) for t in tokens])
    bad = np.nonzero((flat < 0) | (flat >= vocab_size))[0]
    if bad.size:
        raise StepError(f"token id {int(flat[bad[0]])} is outside the vocabulary [0, {vocab_size})")
    wanted = normalize_want(want, new_tokens)

    cache.reserve(slots, new_tokens)  # raises for unknown or repeated slots and for a full pool
    starts = [cache.length(s) for s in slots]

    n = len(slots)
    cu = np.zeros(n + 1, dtype=np.int32)
    cu[1:] = np.cumsum(new_tokens)
    token_seq = np.repeat(np.arange(n, dtype=np.int32), new_tokens)
    token_pos = np.concatenate([np.arange(s, s + k, dtype=np.int32) for s, k in zip(starts, new_tokens)])
    rows = [int(cu[i]) + int(p) for i, w in enumerate(wanted) for p in w]
    tables = {}
    for g in cache.paged_groups():
        lists = [cache.page_list(g, s) for s in slots]
        width = max(1, max(len(l) for l in lists))
        t = np.zeros((n, width), dtype=np.int32)
        for i, l in enumerate(lists):
            t[i, :len(l)] = l
        tables[g] = t
    return StepPlan(slots=slots, new_tokens=new_tokens, starts=starts, token_ids=flat.astype(np.int32),
                    token_seq=token_seq, token_pos=token_pos, cu_tokens=cu,
                    logit_rows=np.asarray(rows, dtype=np.int32), rows_per_seq=[len(w) for w in wanted],
                    block_tables=tables)
