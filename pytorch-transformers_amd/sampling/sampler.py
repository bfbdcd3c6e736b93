"""Choosing the next token of every sequence of a step, on the GPU.

One kernel per step applies the processors that the generation options switch on, in the
reference's order (src/transformers/generation/utils.py:926-1097), and takes the argmax or a draw
(:3274-3279).  Draws come from a counter-based generator keyed by (seed, sequence id, step), not
from a global generator as in the reference (:3277), so a sequence's tokens do not depend on which
other sequences share its batch.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import ops
from ..config.generation import GenerationConfig
from .ahead import TokensAhead
from .bans import BanRules, BiasRules


class Sampler:
    def __init__(self, config: GenerationConfig, vocab_size: int, device):
        self.config = config
        self.vocab_size = vocab_size
        self.device = torch.device(device)
        self.eos_ids = [e for e in config.eos_token_ids]
        self._eos_dev = (torch.tensor(self.eos_ids, dtype=torch.int32, device=self.device)
                         if self.eos_ids else None)
        c = config
        self.do_sample = bool(c.do_sample)
        self.temperature = float(c.temperature) if (c.do_sample and c.temperature is not None) else 1.0
        self.top_k = int(c.top_k) if (c.do_sample and c.top_k) else 0
        self.top_p = float(c.top_p) if (c.do_sample and c.top_p is not None) else 1.0
        self.min_p = float(c.min_p) if (c.do_sample and c.min_p is not None) else 0.0
        self.typical_p = float(c.typical_p) if (c.do_sample and c.typical_p is not None and c.typical_p < 1.0) else 1.0
        # the cut-offs apply strictly between 0 and 1 (src/transformers/generation/utils.py:1076-1087)
        self.epsilon_cutoff = float(c.epsilon_cutoff) if (c.do_sample and c.epsilon_cutoff and 0.0 < c.epsilon_cutoff < 1.0) else 0.0
        self.eta_cutoff = float(c.eta_cutoff) if (c.do_sample and c.eta_cutoff and 0.0 < c.eta_cutoff < 1.0) else 0.0
        self.penalty = float(c.repetition_penalty) if c.repetition_penalty is not None else 1.0
        self.bans = BanRules(c.no_repeat_ngram_size, c.bad_words_ids, c.suppress_tokens, c.begin_suppress_tokens,
                             self.eos_ids)
        self.biases = BiasRules(c.sequence_bias, vocab_size)
        forced = c.forced_eos_token_ids
        self._forced_dev = torch.tensor(forced, dtype=torch.int32, device=self.device) if forced else None
        self.decay = c.exponential_decay_length_penalty  # (start index, factor) or None
        if self.decay is not None and not self.eos_ids:
            raise ValueError("`exponential_decay_length_penalty` raises the scores of the EOS tokens: set `eos_token_id`")

    def step_extras(self, step: int, new_budget: int) -> dict:
        """What ``sample`` needs to know of a step beyond its rows, from the step's number among the new tokens (0
        for the first) and the number of new tokens allowed: whether the last token is forced now
        (src/transformers/generation/logits_process.py:1590-1596: at ``max_length - 1``) and the factor of the
        bonus on EOS (:1716-1727: ``factor ** (tokens past the start index) - 1``, from the token after it)."""
        out = {}
        if self._forced_dev is not None and step == new_budget - 1:
            out["force"] = True
        if self.decay is not None and step > int(self.decay[0]):
            out["decay"] = float(self.decay[1]) ** (step - int(self.decay[0])) - 1.0
        return out

    def sample(self, logits: torch.Tensor, *, rng_seq: Sequence[int], rng_step: Sequence[int],
               histories: Optional[Sequence[Sequence[int]]] = None, suppress_eos: Optional[Sequence[bool]] = None,
               uniforms: Optional[Sequence[float]] = None, new_counts: Optional[Sequence[int]] = None,
               need_scores: bool = True, ahead: bool = False, force: bool = False, decay: Optional[float] = None,
               extra_processors: Optional[Sequence] = None, pad_token_id: Optional[int] = None):
        """Tokens for the rows of ``logits`` and the processed scores ``[rows, vocab]`` (None if not needed
        and the choice could be made without forming them).  ``histories`` are the rows' ids so far (prompt and
        new tokens) and ``new_counts`` how many of them are new; the repetition penalty and the options that forbid
        tokens read them.  ``ahead``: the tokens come back as a ``TokensAhead``, without a wait for the GPU
        (only where ``needs_histories`` is false).

        ``extra_processors``: the caller's own processors, each called as ``processor(input_ids, scores) -> scores``
        with the rows' ids so far as one tensor, padded on the left with ``pad_token_id``, and the scores ``[rows,
        vocab]`` in 32-bit on the device.  They run where the reference puts them: behind the processors that the
        options switch on and in front of temperature, the top-k / top-p family and the renormalization
        (src/transformers/generation/utils.py:1038-1039), which then takes two launches instead of one."""
        R = logits.shape[0]
        if extra_processors:
            if histories is None:
                raise ValueError("the caller's processors are given the rows' ids so far: histories are needed")
            if ahead:
                raise ValueError("tokens ahead of the host cannot pass through the caller's processors")
        if ahead and self.needs_histories:
            raise ValueError("tokens ahead of the host cannot be chosen by options that read the tokens so far")
        suppress = self._eos_dev is not None and suppress_eos is not None and any(suppress_eos)
        ban_lists = None
        force = bool(force) and self._forced_dev is not None
        if self.bans:
            if histories is None:
                raise ValueError("options that forbid tokens by what was generated need the rows' histories")
            counts = new_counts if new_counts is not None else [1] * R
            if force:  # what the forced token overrides does not apply in this step
                ban_lists = [self.bans.banned_after_force(n) for n in counts]
            else:
                ban_lists = [self.bans.banned(h, n) for h, n in zip(histories, counts)]
            if not any(ban_lists):
                ban_lists = None
        bias_lists = None
        if self.biases:
            if histories is None and self.biases.needs_history:
                raise ValueError("a bias on sequences of several tokens needs the rows' histories")
            bias_lists = [self.biases.biases(histories[r] if histories is not None else None) for r in range(R)]
        if (not need_scores and not self.do_sample and self.penalty == 1.0 and not suppress and ban_lists is None
                and not self.config.remove_invalid_values and not self.config.renormalize_logits
                and bias_lists is None and not force and decay is None and not extra_processors):
            # greedy with no processor in the way: nothing to upload, one argmax kernel
            chosen = ops.sample(logits, do_sample=False, need_scores=False)[0]
            return (TokensAhead(chosen) if ahead else chosen.tolist()), None
        use_hist = self.penalty != 1.0 and histories is not None
        pieces = [np.asarray(rng_seq, dtype=np.int32), np.asarray(rng_step, dtype=np.int32),
                  np.asarray([1 if s else 0 for s in (suppress_eos or [False] * R)], dtype=np.int32)]
        if use_hist:
            off = np.zeros(R + 1, dtype=np.int32)
            off[1:] = np.cumsum([len(h) for h in histories])
            flat = (np.concatenate([np.asarray(h, dtype=np.int32) for h in histories])
                    if off[-1] else np.zeros(0, dtype=np.int32))
            pieces += [off, flat]
        n_before = len(pieces)
        if ban_lists is not None:
            boff = np.zeros(R + 1, dtype=np.int32)
            boff[1:] = np.cumsum([len(b) for b in ban_lists])
            pieces += [boff, np.asarray([t for b in ban_lists for t in b], dtype=np.int32)]
        n_bias_at = len(pieces)
        if bias_lists is not None:  # offsets, tokens, and the values' bits as integers (one buffer, one copy)
            voff = np.zeros(R + 1, dtype=np.int32)
            voff[1:] = np.cumsum([len(b) for b in bias_lists])
            pieces += [voff, np.asarray([t for b in bias_lists for t, _ in b], dtype=np.int32),
                       np.asarray([v for b in bias_lists for _, v in b], dtype=np.float32).view(np.int32)]
        staged = torch.from_numpy(np.concatenate(pieces))
        # (ahead of the host nothing may wait for the stream: the copy starts from pinned memory and does not block)
        dev = staged.pin_memory().to(self.device, non_blocking=True) if ahead else staged.to(self.device)
        views = torch.split(dev, [int(p.shape[0]) for p in pieces])
        if uniforms is None:
            u = None
        elif ahead:
            u = torch.tensor(list(uniforms), dtype=torch.float32).pin_memory().to(self.device, non_blocking=True)
        else:
            u = torch.tensor(list(uniforms), dtype=torch.float32, device=self.device)
        warpers = dict(do_sample=self.do_sample, temperature=self.temperature, top_k=self.top_k, top_p=self.top_p,
                       min_p=self.min_p, typical_p=self.typical_p, epsilon_cutoff=self.epsilon_cutoff,
                       eta_cutoff=self.eta_cutoff, renorm=self.config.renormalize_logits)
        draws = dict(seed=self.config.seed, rng_seq=views[0], rng_step=views[1], uniforms=u)
        processors = dict(
            penalty=self.penalty, hist=views[4] if use_hist else None,
            hist_off=views[3] if use_hist else None, ban=views[n_before + 1] if ban_lists is not None else None,
            ban_off=views[n_before] if ban_lists is not None else None, eos=self._eos_dev,
            suppress=views[2] if (self._eos_dev is not None and suppress_eos is not None and any(suppress_eos)) else None,
            remove_invalid=self.config.remove_invalid_values,
            bias_off=views[n_bias_at] if bias_lists is not None else None,
            bias_tok=views[n_bias_at + 1] if bias_lists is not None else None,
            bias_val=views[n_bias_at + 2].view(torch.float32) if bias_lists is not None else None,
            forced=self._forced_dev if force else None, decay=decay)
        if not extra_processors:
            tokens, scores = ops.sample(logits, need_scores=need_scores, **warpers, **draws, **processors)
        else:
            # the options' processors alone (the greedy form of the launch returns their scores untouched by any
            # warper), the caller's on that tensor, then the warpers and the choice
            _, scores = ops.sample(logits, do_sample=False, need_scores=True, **draws, **processors)
            ids = left_padded(histories, 0 if pad_token_id is None else int(pad_token_id), self.device)
            for proc in extra_processors:
                scores = proc(ids, scores)
                if not (isinstance(scores, torch.Tensor) and scores.shape == logits.shape):
                    raise ValueError(f"the processor {proc!r} must return scores of shape {tuple(logits.shape)}")
            scores = scores.to(device=self.device, dtype=torch.float32).contiguous()
            tokens, scores = ops.sample(scores, need_scores=need_scores, **warpers, **draws)
        return (TokensAhead(tokens) if ahead else tokens.tolist()), scores

    @property
    def needs_histories(self) -> bool:
        """Whether a choice reads the sequence's tokens so far (which the host then has to have seen)."""
        return bool(self.bans) or self.penalty != 1.0 or self.biases.needs_history


def left_padded(histories: Sequence[Sequence[int]], pad: int, device) -> torch.Tensor:
    """The rows' ids as the reference's rectangular ``input_ids``: int64 ``[rows, longest]``, shorter rows padded on
    the left."""
    longest = max(len(h) for h in histories)
    ids = np.full((len(histories), longest), int(pad), dtype=np.int64)
    for r, h in enumerate(histories):
        if len(h):
            ids[r, longest - len(h):] = np.asarray(h, dtype=np.int64)
    return torch.from_numpy(ids).to(device)


def philox_uniform(seed: int, seq: int, step: int) -> float:
    """The uniform number in [0, 1) that the kernel draws for (seed, sequence id, step)."""
    lib = ops.load_library()
    lib.pta_philox_uniform.restype = ctypes.c_float
    return float(lib.pta_philox_uniform(ctypes.c_uint64(seed & (2 ** 64 - 1)), ctypes.c_uint32(seq), ctypes.c_uint32(step)))
