"""Tokens that a sequence may not take next, decided on the host from its ids so far.

The kernel takes a list of banned ids per row and sets their scores to -inf; this module makes that list
from the options that forbid tokens by what has been generated:

* ``no_repeat_ngram_size = n``: a token that would complete an n-gram that the sequence already holds
  (src/transformers/generation/logits_process.py:840-903, :954-962).  The reference looks through the
  padded row, this one through the sequence's own ids: padding never takes part in an n-gram here.
* ``bad_words_ids``: a one-token entry is always banned, a longer one bans its last token while the
  sequence ends in the tokens before it (:1110-1140, :1270-1286; an entry that is just an EOS token is
  dropped, :1272-1282).
* ``suppress_tokens``: always banned (:1853-1857).
* ``begin_suppress_tokens``: banned for the first generated token only (:1810-1817).

All of them write -inf, so their order among each other and with the repetition penalty (which scales a
score and leaves -inf where it is) does not matter.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np


def repeated_ngram_tokens(ids: Sequence[int], n: int) -> List[int]:
    """Tokens that followed an earlier occurrence of the last ``n - 1`` ids (every token that occurred, for n = 1)."""
    if n <= 0 or len(ids) + 1 < n:
        return []
    a = np.asarray(ids, dtype=np.int64)
    if n == 1:
        return sorted(set(a.tolist()))
    tail = a[len(a) - (n - 1):]
    starts = len(a) - (n - 1)  # an earlier occurrence at j needs a token after it: j + n - 1 <= len - 1
    hit = np.ones(starts, dtype=bool)
    for k in range(n - 1):
        hit &= a[k:k + starts] == tail[k]
    return sorted(set(a[np.nonzero(hit)[0] + (n - 1)].tolist()))


def bad_word_tokens(ids: Sequence[int], bad_words: Sequence[Sequence[int]]) -> List[int]:
    out = set()
    for word in bad_words:
        k = len(word) - 1
        if k == 0 or (k <= len(ids) and list(ids[len(ids) - k:]) == list(word[:-1])):
            out.add(int(word[-1]))
    return sorted(out)


class BanRules:
    """The options of one generation call that forbid tokens; ``banned(ids, n_new)`` is a sequence's list."""

    def __init__(self, no_repeat_ngram_size: Optional[int] = None, bad_words_ids=None, suppress_tokens=None,
                 begin_suppress_tokens=None, eos_token_ids: Sequence[int] = ()):
        self.ngram = int(no_repeat_ngram_size or 0)
        eos = set(int(e) for e in eos_token_ids)
        self.bad_words = [list(w) for w in (bad_words_ids or []) if not (len(w) == 1 and int(w[0]) in eos)]
        self.always = sorted(set(int(t) for t in (suppress_tokens or [])))
        self.begin = sorted(set(int(t) for t in (begin_suppress_tokens or [])))

    def __bool__(self) -> bool:
        return bool(self.ngram or self.bad_words or self.always or self.begin)

    def banned(self, ids: Sequence[int], n_new: int) -> List[int]:
        out = set(self.always)
        if self.begin and n_new == 0:
            out.update(self.begin)
        if self.ngram:
            out.update(repeated_ngram_tokens(ids, self.ngram))
        if self.bad_words:
            out.update(bad_word_tokens(ids, self.bad_words))
        return sorted(out)
