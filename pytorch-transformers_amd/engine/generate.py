"""The generation loop: batches of unequal prompts, stop tokens, sequences that end earlier.

What the reference's ``generate`` and ``_sample`` do
(src/transformers/generation/utils.py:1908-2401, :3139-3324), on top of the step function:

* prompts of a batch go through one step together, unpadded, then every live sequence brings one
  token per step; the reference pads on the left and masks (:2036-2059);
* a sequence that produced a stop token (kept in its output, stopping_criteria.py:446-467) or
  reached its length leaves the batch and gives its slot back at once; the reference keeps
  feeding it padding until all rows are done (:3282-3291);
* requests beyond ``batch_size`` run as further batches on the same cache, whose slots and pages
  are used again.

The loop decides on the host and needs from the model only ``new_cache``, ``step`` and a sampler,
so its decisions are tested without a GPU.
"""
from __future__ import annotations

import dataclasses
import time
from typing import List, Optional, Sequence, Union

from ..config.generation import GenerationConfig


@dataclasses.dataclass
class GenerateOutput:
    """``return_dict_in_generate=True`` (src/transformers/generation/utils.py:3314-3322)."""

    sequences: List[List[int]]
    scores: Optional[List[List]] = None  # per sequence, per new token: processed scores [vocab]
    logits: Optional[List[List]] = None  # per sequence, per new token: raw logits [vocab]
    #: with ``keep_slots``: the cache that holds the sequences and each sequence's slot in it, for a later call
    #: that goes on from there (the reference returns ``past_key_values`` for that, :3314-3322)
    cache: Optional[object] = None
    slots: Optional[List[int]] = None
    #: with ``keep_slots``: per sequence, how many draws of its random stream are used up (``rng_step_start`` of the
    #: call that goes on, so that it draws what one call over the whole length would have drawn)
    rng_steps: Optional[List[int]] = None


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


def resolve_lengths(cfg: GenerationConfig, prompt_lens: Sequence[int]):
    """New tokens per sequence and the padded length the reference's length rules count from.

    ``max_new_tokens`` wins over ``max_length`` (:1461); the reference measures lengths on the
    left-padded batch, so every row gets the same number of new tokens; a prompt that already
    fills ``max_length`` is an error (:1409-1415).
    """
    longest = max(prompt_lens)
    if cfg.max_new_tokens is not None:
        new = int(cfg.max_new_tokens)
    else:
        new = int(cfg.max_length) - longest
        if new <= 0:
            raise ValueError(
                f"Input length of input_ids is {longest}, but `max_length` is set to {cfg.max_length}. This can "
                "lead to unexpected behavior. You should consider increasing `max_length` or, better yet, setting "
                "`max_new_tokens`.")
    return new, longest


def generate(model, prompts: Sequence[Sequence[int]], generation_config: Optional[GenerationConfig] = None, *,
             batch_size: Optional[int] = None, sampler=None, streamer=None, cache=None,
             rng_ids: Optional[Sequence[int]] = None, tokenizer=None, keep_slots: bool = False,
             slots: Optional[Sequence[int]] = None, rng_step_start: Optional[Sequence[int]] = None,
             logits_processor: Optional[Sequence] = None, stopping_criteria: Optional[Sequence] = None,
             attention_mask=None, **kwargs) -> Union[List[List[int]], GenerateOutput]:
    """Generate for every prompt (a list of token ids); returns prompt + new tokens per prompt.

    ``prompts`` may also be the reference's rectangular ``input_ids``, an integer tensor ``[rows, longest]`` with
    ``attention_mask`` (same shape; 0 where a row is padded, on the left as the reference asks of decoder-only
    models, src/transformers/generation/utils.py:2036-2048): a row's prompt is then its ids where the mask is 1, and the
    result is the reference's tensor, prompts padded on the left and finished rows on the right with
    ``pad_token_id`` (the first ``eos_token_id`` if there is none, :1863-1871; ``sequences`` of a ``GenerateOutput``
    likewise).

    ``generation_config`` defaults to the model's; keyword arguments override its fields
    (:1543-1545).  ``streamer``: an object with ``put`` and ``end`` as the reference's streamers have them
    (src/transformers/generation/streamers.py:23-39: ``put`` is given the prompt first and then every new token, one
    prompt per call; src/transformers/generation/utils.py:2087, :3288, :3301-3302), or a callable ``streamer(index, token)`` for any number of prompts
    (and ``streamer.end()`` if it has one).  ``logits_processor``: the caller's own processors, ``processor(input_ids,
    scores) -> scores``, run behind those that the options switch on and in front of temperature and the top-k
    family (:1038-1039); ``stopping_criteria``: ``criterion(input_ids, scores)`` gives a flag per row (or one for
    all), and a row whose flag is set ends with the token just chosen (:1136, stopping_criteria.py:491-497).  Both
    are handed the rows' ids so far as one int64 tensor, padded on the left with ``pad_token_id`` (0 if none).  ``rng_ids`` name each prompt's random stream (default: its
    index), so that a prompt draws the same tokens in any batch.  ``tokenizer`` (anything with
    ``decode(ids) -> str``) is needed for ``stop_strings`` only: a sequence ends with the token that
    completes one of them in the text of its new tokens (src/transformers/generation/utils.py:1118-1125,
    stopping_criteria.py:110-443; the token is kept, as the reference keeps it).

    ``keep_slots``: sequences keep their cache slots when they end instead of giving them back, and the result
    is a ``GenerateOutput`` with ``cache`` and ``slots``.  A later call goes on from there when it is given that
    cache, those ``slots`` and, as prompts, the whole sequences so far: only the tokens a slot does not hold yet
    are run (the reference continues from a returned cache the same way, src/transformers/generation/utils.py
    :349-481, tests/generation/test_utils.py:1775-1855).  Whoever keeps slots frees them (``cache.free``), or
    hands them to a call without ``keep_slots``, which frees them when it ends.  A random stream is a sequence of
    draws numbered from 0; ``rng_step_start`` says, per prompt, at which number this call starts (default 0).  A call
    that goes on from kept slots passes the earlier result's ``rng_steps`` there and then samples the tokens that
    one call over the whole length would have sampled.
    """
    cfg = generation_config or getattr(model, "generation_config", None) or GenerationConfig()
    if kwargs:
        cfg = cfg.updated(**kwargs)
    if hasattr(prompts, "dim"):  # a tensor: the reference's input_ids
        return _generate_from_tensor(model, prompts, attention_mask, cfg, dict(
            batch_size=batch_size, sampler=sampler, streamer=streamer, cache=cache, rng_ids=rng_ids, tokenizer=tokenizer,
            keep_slots=keep_slots, slots=slots, rng_step_start=rng_step_start, logits_processor=logits_processor,
            stopping_criteria=stopping_criteria))
    if attention_mask is not None:
        raise ValueError("an attention_mask goes with input_ids as a tensor; prompts given as lists have no padding")
    prompts = [list(map(int, p)) for p in prompts]
    if not prompts:
        return GenerateOutput([]) if cfg.return_dict_in_generate else []
    bos = cfg.bos_token_id
    for i, p in enumerate(prompts):
        if not p:  # an empty prompt starts from BOS (:547-577)
            if bos is None:
                raise ValueError(f"prompt {i} is empty and no bos_token_id is set")
            prompts[i] = [int(bos)]
    n_ret = cfg.num_return_sequences
    if slots is not None:
        slots = [int(s_) for s_ in slots]
        if cache is None:
            raise ValueError("slots to go on from need the cache they live in")
        if n_ret > 1:
            raise ValueError("a call that goes on from kept slots returns one sequence per slot")
        if len(slots) != len(prompts) or len(set(slots)) != len(slots):
            raise ValueError(f"{len(prompts)} prompts but slots {slots}: one slot of its own per prompt")
        for p, s_ in zip(prompts, slots):
            held = cache.length(s_)
            if held >= len(p):
                raise ValueError(f"slot {s_} already holds {held} tokens, the sequence given for it has {len(p)}: "
                                 "give the whole sequence so far, which ends with a token that has not been run yet")
    if n_ret > 1:  # :2244-2249, :716-748
        prompts = [p for p in prompts for _ in range(n_ret)]
    ids = list(rng_ids) if rng_ids is not None else list(range(len(prompts)))
    if n_ret > 1 and rng_ids is not None:
        ids = [r * n_ret + j for r in rng_ids for j in range(n_ret)]
    if len(ids) != len(prompts):
        raise ValueError("rng_ids must name one stream per prompt")
    first_draw = [int(v) for v in rng_step_start] if rng_step_start is not None else [0] * (len(prompts) // n_ret)
    if len(first_draw) * n_ret != len(prompts) or any(v < 0 for v in first_draw):
        raise ValueError("rng_step_start must give one number, 0 or more, per prompt")
    first_draw = [v for v in first_draw for _ in range(n_ret)]

    batch_size = batch_size or len(prompts)
    batches = [list(range(b, min(b + batch_size, len(prompts)))) for b in range(0, len(prompts), batch_size)]
    page = cache.page_size if cache is not None else getattr(model, "page_size", 64)
    per_batch = []
    for b in batches:
        new, _ = resolve_lengths(cfg, [len(prompts[i]) for i in b])
        per_batch.append(sum(_round_up(len(prompts[i]) + new, page) for i in b))
    if cache is None:  # kept slots stay held while later batches run
        cache = model.new_cache(sum(per_batch) if keep_slots else max(per_batch),
                                max_slots=len(prompts) if keep_slots else batch_size)
    if sampler is None:
        from ..sampling.sampler import Sampler

        sampler = Sampler(cfg, model.vocab_size, model.device)

    eos = set(cfg.eos_token_ids)
    stop_strings = [cfg.stop_strings] if isinstance(cfg.stop_strings, str) else list(cfg.stop_strings or [])
    if stop_strings and tokenizer is None:
        raise ValueError(
            "There are one or more stop strings, either in the arguments to `generate` or in the model's generation "
            "config, but we could not locate a tokenizer. When generating with stop strings, you must pass the model's "
            "tokenizer to the `tokenizer` argument of `generate`.")
    logits_processor, stopping_criteria = list(logits_processor or []), list(stopping_criteria or [])
    puts = streamer is not None and hasattr(streamer, "put")
    if puts and len(prompts) != 1:
        raise ValueError("TextStreamer only supports batch size 1")  # streamers.py:87-88
    want_scores, want_logits = bool(cfg.output_scores), bool(cfg.output_logits)
    out_tokens: List[List[int]] = [[] for _ in prompts]
    out_scores = [[] for _ in prompts] if want_scores else None
    out_logits = [[] for _ in prompts] if want_logits else None
    kept = [None] * len(prompts)
    t0 = time.time()
    # Steps ahead of the host: where nothing of a step's decisions needs more than the tokens themselves, the next
    # step is launched from the tokens on the device before the host has read them.
    ahead = (bool(getattr(model, "steps_ahead", False)) and getattr(sampler, "needs_histories", True) is False
             and not want_scores and not want_logits and streamer is None and not stop_strings
             and cfg.max_time is None and not keep_slots and not logits_processor and not stopping_criteria)
    pad = 0 if cfg.pad_token_id is None else int(cfg.pad_token_id)
    custom = dict(extra_processors=logits_processor, pad_token_id=pad) if logits_processor else {}
    if puts:
        streamer.put(_ids_tensor(prompts[0]))

    def done_with(i: int, slot: int) -> None:
        if keep_slots:
            kept[i] = slot
        else:
            cache.free(slot)

    for batch in batches:
        new_budget, padded_len = resolve_lengths(cfg, [len(prompts[i]) for i in batch])
        if slots is not None:  # going on: each sequence's slot holds its first tokens already
            slot_of = {i: slots[i] for i in batch}
            feed = {i: prompts[i][cache.length(slots[i]):] for i in batch}
        else:
            slot_of = {i: cache.alloc() for i in batch}
            feed = {i: prompts[i] for i in batch}
        live = list(batch)
        step_no = 0
        try:
            if ahead:
                _decode_ahead(model, cache, sampler, cfg, eos, ids, batch, slot_of, feed, out_tokens, new_budget,
                              padded_len, done_with, first_draw)
                live = []
            while live:
                logits = model.step(cache, [slot_of[i] for i in live], [feed[i] for i in live], "last")
                # EOS is masked while the minimum lengths are not reached (logits_process.py:144-151, :214-223)
                too_short = (padded_len + step_no < (cfg.min_length or 0)) or (step_no < (cfg.min_new_tokens or 0))
                tokens, scores = sampler.sample(
                    logits, rng_seq=[ids[i] for i in live], rng_step=[first_draw[i] + step_no for i in live],
                    histories=[prompts[i] + out_tokens[i] for i in live], suppress_eos=[too_short] * len(live),
                    new_counts=[len(out_tokens[i]) for i in live],
                    need_scores=want_scores or bool(stopping_criteria), **custom,
                    **_step_extras(sampler, step_no, new_budget))
                step_no += 1
                timed_out = cfg.max_time is not None and (time.time() - t0) > cfg.max_time  # stopping_criteria.py:87-107
                still = []
                for row, i in enumerate(live):
                    out_tokens[i].append(int(tokens[row]))
                halted = _criteria_flags(stopping_criteria, [prompts[i] + out_tokens[i] for i in live], scores, pad)
                for row, i in enumerate(live):
                    tok = out_tokens[i][-1]
                    if want_scores:
                        out_scores[i].append(scores[row].clone())
                    if want_logits:
                        out_logits[i].append(logits[row].clone())
                    if puts:
                        streamer.put(_ids_tensor([tok]))
                    elif streamer is not None:
                        streamer(i, tok)
                    said_stop = bool(stop_strings) and _ends_with_stop(tokenizer, out_tokens[i], stop_strings)
                    if tok in eos or step_no >= new_budget or timed_out or said_stop or halted[row]:
                        done_with(i, slot_of.pop(i))
                    else:
                        feed[i] = [tok]
                        still.append(i)
                live = still
        except BaseException:
            for i in list(slot_of):  # a step failed: nothing of this batch can be gone on from
                cache.free(slot_of.pop(i))
            for i, slot in enumerate(kept):  # nor of the earlier batches: the caller never learns their slots
                if slot is not None:
                    cache.free(slot)
                    kept[i] = None
            raise
    if streamer is not None and hasattr(streamer, "end"):
        streamer.end()
    sequences = [p + t for p, t in zip(prompts, out_tokens)]
    if keep_slots:
        return GenerateOutput(sequences, out_scores, out_logits, cache=cache, slots=kept,
                              rng_steps=[first_draw[i] + len(out_tokens[i]) for i in range(len(prompts))])
    if cfg.return_dict_in_generate:
        return GenerateOutput(sequences, out_scores, out_logits)
    return sequences


def _generate_from_tensor(model, input_ids, attention_mask, cfg: GenerationConfig, how: dict):
    """``generate`` for the reference's rectangular input: rows without their padding in, the reference's tensor out."""
    import torch

    if input_ids.dim() != 2 or input_ids.dtype not in (torch.int64, torch.int32):
        raise ValueError(f"input_ids must be an integer tensor [rows, length], got {tuple(input_ids.shape)} {input_ids.dtype}")
    ids = input_ids.detach().cpu()
    if attention_mask is None:
        rows = ids.tolist()
    else:
        mask = torch.as_tensor(attention_mask).detach().cpu()
        if mask.shape != ids.shape:
            raise ValueError(f"attention_mask {tuple(mask.shape)} must have the shape of input_ids {tuple(ids.shape)}")
        rows = [r[m.bool()].tolist() for r, m in zip(ids, mask)]
    out = generate(model, rows, cfg, **how)
    pad = cfg.pad_token_id
    if pad is None:
        pad = cfg.eos_token_ids[0] if cfg.eos_token_ids else 0
    n_ret = cfg.num_return_sequences
    lens = [len(r) for r in rows for _ in range(n_ret)]
    seqs = out.sequences if isinstance(out, GenerateOutput) else out
    padded = pad_sequences(seqs, lens, pad).to(input_ids.device)
    if isinstance(out, GenerateOutput):
        out.sequences = padded
        return out
    return padded


def _ids_tensor(ids: Sequence[int]):
    import torch

    return torch.tensor(list(ids), dtype=torch.long)


def _criteria_flags(criteria: Sequence, sequences: Sequence[Sequence[int]], scores, pad: int) -> List[bool]:
    """Which of the rows the caller's stopping criteria end now: each criterion is called with the rows' ids (the
    token just chosen included) and the step's scores, and gives a flag per row or one for all rows; a row ends if
    any criterion says so (src/transformers/generation/stopping_criteria.py:491-497)."""
    flags = [False] * len(sequences)
    if not criteria:
        return flags
    import torch

    from ..sampling.sampler import left_padded

    ids = left_padded(sequences, pad, scores.device if scores is not None else "cpu")
    for criterion in criteria:
        said = criterion(ids, scores)
        said = said.reshape(-1).tolist() if isinstance(said, torch.Tensor) else [bool(said)]
        if len(said) == 1:
            said = said * len(sequences)
        if len(said) != len(sequences):
            raise ValueError(f"the stopping criterion {criterion!r} gave {len(said)} flags for {len(sequences)} rows")
        flags = [a or bool(b) for a, b in zip(flags, said)]
    return flags


def _step_extras(sampler, step: int, new_budget: int) -> dict:
    """The processors that follow the step's number rather than its rows (a forced last token, the bonus on EOS that
    grows with the length), for samplers that have them."""
    extras = getattr(sampler, "step_extras", None)
    return extras(step, new_budget) if extras is not None else {}


def _decode_ahead(model, cache, sampler, cfg, eos, ids, batch, slot_of, feed, out_tokens, new_budget, padded_len,
                  done_with, first_draw) -> None:
    """One batch, with every step launched before the host has seen the tokens of the step before it.

    The tokens of a step stay on the device (``sampler.sample(..., ahead=True)``) and the next step takes them
    from there (``model.step`` with those tokens); while it runs the host reads the earlier tokens, appends them
    and finds who has ended.  A sequence that ended on a stop token was part of one more step, whose row nobody
    reads: its keys and values went into a slot that is given back, and whatever takes the slot's pages next is
    launched later on the same stream.  A sequence that ends by its length is known beforehand and never takes
    part in a step too many.  The tokens are those of the loop that waits after every step: a sequence's result
    does not depend on what else is in its batch.
    """
    from ..cache.paged import CacheFull

    def too_short(step: int) -> bool:  # as in the loop that waits: EOS is masked until the minimum lengths are reached
        return (padded_len + step < (cfg.min_length or 0)) or (step < (cfg.min_new_tokens or 0))

    def choose(logits, seqs, step):
        return sampler.sample(logits, rng_seq=[ids[i] for i in seqs], rng_step=[first_draw[i] + step for i in seqs],
                              suppress_eos=[too_short(step)] * len(seqs), need_scores=False, ahead=True,
                              **_step_extras(sampler, step, new_budget))[0]

    step_no = 0  # the number of the token that `pending` holds for each of its sequences
    seqs = list(batch)
    pending = choose(model.step(cache, [slot_of[i] for i in seqs], [feed[i] for i in seqs], "last"), seqs, 0)
    rows = list(range(len(seqs)))  # the rows of `pending` whose sequences live, as far as the host knows
    while True:
        nxt = None
        if step_no + 1 < new_budget:  # (else every sequence ends with the pending token)
            try:
                logits = model.step(cache, [slot_of[i] for i in seqs], pending.take(rows), "last", own_logits=False)
            except CacheFull:
                logits = None  # no room to go on before knowing who has ended: wait for the tokens first
            if logits is not None:
                nxt = choose(logits, seqs, step_no + 1)
        tokens = pending.tolist()
        step_no += 1
        on = []  # of the next step's rows, those whose sequences go on
        for at, (row, i) in enumerate(zip(rows, seqs)):
            tok = int(tokens[row])
            out_tokens[i].append(tok)
            if tok in eos or step_no >= new_budget:
                done_with(i, slot_of.pop(i))
            else:
                on.append(at)
        if not on:
            return
        survivors = [seqs[at] for at in on]
        if nxt is None:  # the step that found no room: now with the sequences that are left, and their tokens
            logits = model.step(cache, [slot_of[i] for i in survivors], [[out_tokens[i][-1]] for i in survivors], "last")
            pending, rows = choose(logits, survivors, step_no), list(range(len(survivors)))
        else:
            pending, rows = nxt, on
        seqs = survivors


def _ends_with_stop(tokenizer, new_tokens: Sequence[int], stop_strings: Sequence[str]) -> bool:
    """Whether the last token completed a stop string: the string lies in the text of the new tokens and not
    wholly in the text before the last token."""
    text = tokenizer.decode(list(new_tokens))
    before = tokenizer.decode(list(new_tokens[:-1])) if len(new_tokens) > 1 else ""
    return any(s and s in text and s not in before for s in stop_strings)


def compute_transition_scores(output: "GenerateOutput", prompt_lens: Sequence[int], normalize_logits: bool = False):
    """The score of every generated token: per sequence, ``scores[step][token chosen at that step]`` from a result
    of ``generate(..., output_scores=True, return_dict_in_generate=True)`` (src/transformers/generation/utils.py
    :1160-1283 without beams); with ``normalize_logits`` the log-softmax of the step's scores first.  Sequences are
    ragged here (one that ended early has fewer steps), so the result is a list of 32-bit tensors, one per sequence."""
    import torch

    if output.scores is None:
        raise ValueError("transition scores need the steps' scores: generate(..., output_scores=True)")
    out = []
    for seq, n, steps in zip(output.sequences, prompt_lens, output.scores):
        new = [int(t) for t in (seq.tolist() if hasattr(seq, "tolist") else seq)][int(n):int(n) + len(steps)]
        vals = []
        for tok, s in zip(new, steps):
            s = s.float()
            vals.append((torch.log_softmax(s, -1) if normalize_logits else s)[tok])
        out.append(torch.stack(vals) if vals else torch.zeros(0))
    return out


def pad_sequences(sequences: Sequence[Sequence[int]], prompt_lens: Sequence[int], pad_token_id: int):
    """The reference's rectangular return value: prompts padded on the left to the longest prompt, new
    tokens padded on the right after a row ended (src/transformers/generation/utils.py:3282-3286)."""
    import torch

    longest = max(prompt_lens)
    width = longest + max(len(s) - n for s, n in zip(sequences, prompt_lens))
    out = torch.full((len(sequences), width), int(pad_token_id), dtype=torch.long)
    for r, (s, n) in enumerate(zip(sequences, prompt_lens)):
        out[r, longest - n:longest - n + len(s)] = torch.as_tensor(list(s), dtype=torch.long)
    return out
