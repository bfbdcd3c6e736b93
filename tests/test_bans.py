"""The host's decision which tokens a sequence may not take next (no GPU)."""
import random

import pytest

from pytorch_transformers_amd.config import GenerationConfig
from pytorch_transformers_amd.sampling.bans import BanRules, bad_word_tokens, repeated_ngram_tokens


def test_no_repeat_ngram_reference_vectors():
    """tests/generation/test_logits_process.py:485-508."""
    assert repeated_ngram_tokens([1, 1, 2, 1], 2) == [1, 2]
    assert repeated_ngram_tokens([0, 1, 0, 1], 2) == [0]
    assert repeated_ngram_tokens([1, 1, 2, 1], 3) == []
    assert repeated_ngram_tokens([0, 1, 0, 1], 3) == [0]
    assert repeated_ngram_tokens([5], 3) == [] and repeated_ngram_tokens([], 1) == []
    assert repeated_ngram_tokens([4, 2, 4], 1) == [2, 4]


def test_no_repeat_ngram_against_a_dictionary_of_ngrams():
    """The definition itself: every n-gram of the sequence, keyed by its first n - 1 tokens
    (src/transformers/generation/logits_process.py:840-903)."""
    rnd = random.Random(3)
    for _ in range(200):
        n = rnd.randint(1, 4)
        ids = [rnd.randint(0, 4) for _ in range(rnd.randint(0, 30))]
        follows = {}
        for j in range(len(ids) - n + 1):
            follows.setdefault(tuple(ids[j:j + n - 1]), set()).add(ids[j + n - 1])
        want = sorted(follows.get(tuple(ids[len(ids) - (n - 1):]) if n > 1 else (), set())) if len(ids) + 1 >= n else []
        assert repeated_ngram_tokens(ids, n) == want, (ids, n)


def test_bad_words_reference_vectors():
    """tests/generation/test_logits_process.py:576-601: one-token entries always, longer ones when the sequence
    ends in their first tokens; an entry that is the EOS token alone is dropped."""
    rules = BanRules(bad_words_ids=[[1], [4], [1, 0], [0, 1, 2], [1, 3, 1, 3]], eos_token_ids=[4])
    assert rules.banned([0, 1, 3, 1], 1) == [0, 1, 3]
    assert rules.banned([0, 1, 0, 1], 1) == [0, 1, 2]
    assert not BanRules(bad_words_ids=[[4]], eos_token_ids=[4])
    assert bad_word_tokens([7], [[1, 2, 3, 4]]) == []  # an entry longer than the sequence


def test_suppress_tokens_and_the_first_new_token():
    rules = BanRules(suppress_tokens=[9, 3], begin_suppress_tokens=[5])
    assert rules.banned([1, 2], 0) == [3, 5, 9] and rules.banned([1, 2, 4], 1) == [3, 9]
    assert not BanRules() and BanRules(no_repeat_ngram_size=2)


def test_options_are_checked():
    with pytest.raises(ValueError, match="ngram_size"):
        GenerationConfig(no_repeat_ngram_size=-1)
    with pytest.raises(ValueError, match="bad_words_ids"):
        GenerationConfig(bad_words_ids=[])
    with pytest.raises(ValueError, match="bad_words_ids"):
        GenerationConfig(bad_words_ids=[[1, -2]])
    assert GenerationConfig(no_repeat_ngram_size=3, bad_words_ids=[[1, 2]]).no_repeat_ngram_size == 3
