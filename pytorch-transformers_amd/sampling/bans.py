"""Tokens that a sequence may not take next, decided on the host from its ids so far.

The kernel takes a list of banned ids per row and sets their scores to -inf; this module makes that list
from the options that forbid tokens by what has been generated:

* ``no_repeat_ngram_size = n``: a token that would complete an n-gram that the sequence already holds
  (src/transformers/generation/logits_process.py:840-903, :954-962).  The reference looks through the
  padded row, this one through the sequence's own ids: padding never takes part in an n-gram here.
* ``bad_words_ids``: a one-token entry is always banned, a longer one bans its last token while the
  sequence ends in the tokens before it and is at least as long as the entry (:1110-1140, :1270-1286; an
  entry that is just an EOS token is dropped, :1272-1282).
* ``suppress_tokens``: always banned (:1853-1857).
* ``begin_suppress_tokens``: banned for the first generated token only (:1810-1817).

All of them write -inf, so their order among each other and with the repetition penalty (which scales a
score and leaves -inf where it is) does not matter.  One processor stands between them in the reference's order:
a forced last token (``forced_eos_token_id``) comes after the first two and before the last two, and overrides
what came before it, so in a step that forces a token only the last two apply (``banned_after_force``).

``BiasRules`` makes, in the same manner, the list of tokens whose scores get a value added (``sequence_bias``,
:1112-1140): an entry of one token always, a longer one for its last token while the sequence ends in the tokens
before it; entries that end in the same token add up.
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
        # (an entry longer than the ids so far never applies, logits_process.py:1122)
        if k == 0 or (len(word) <= len(ids) and list(ids[len(ids) - k:]) == list(word[:-1])):
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

    def banned_after_force(self, n_new: int) -> List[int]:
        """What is banned in a step that forces a token: the options that come after that in the reference's order."""
        out = set(self.always)
        if self.begin and n_new == 0:
            out.update(self.begin)
        return sorted(out)

    def banned(self, ids: Sequence[int], n_new: int) -> List[int]:
        out = set(self.banned_after_force(n_new))
        if self.ngram:
            out.update(repeated_ngram_tokens(ids, self.ngram))
        if self.bad_words:
            out.update(bad_word_tokens(ids, self.bad_words))
        return sorted(out)


class BiasRules:
    """``sequence_bias`` of one generation call; ``biases(ids)`` is a sequence's list of (token, value), each token once."""

    def __init__(self, sequence_bias=None, vocab_size: Optional[int] = None):
        entries = [(tuple(int(t) for t in e[0]), float(e[1])) for e in (sequence_bias or [])]
        if vocab_size is not None:  # logits_process.py:1148-1158
            beyond = [t for seq, _ in entries for t in seq if t >= vocab_size]
            if beyond:
                raise ValueError(f"The model vocabulary size is {vocab_size}, but the following tokens were being biased: "
                                 f"{beyond}")
        merged = dict(entries)  # an entry given twice counts once, the later value (a dict in the reference, :1216-1220)
        self.single = {seq[0]: v for seq, v in merged.items() if len(seq) == 1}
        self.longer = [(seq, v) for seq, v in merged.items() if len(seq) > 1]

    def __bool__(self) -> bool:
        return bool(self.single or self.longer)

    @property
    def needs_history(self) -> bool:
        return bool(self.longer)

    def biases(self, ids: Optional[Sequence[int]]) -> List[tuple]:
        out = dict(self.single)
        for seq, v in self.longer:
            k = len(seq) - 1
            if ids is not None and len(seq) <= len(ids) and tuple(ids[len(ids) - k:]) == seq[:-1]:
                out[seq[-1]] = out.get(seq[-1], 0.0) + v
        return sorted(out.items())
