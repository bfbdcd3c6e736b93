"""Shared test helpers: requests, replay schedules and comparison with the plain implementation."""
from __future__ import annotations

import random
from typing import Dict, List, Sequence

import torch

import plain_falcon as plain


def make_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


# --- schedules: lists of trace records -------------------------------------------------
def schedule_whole(reqs: Dict[str, List[int]]) -> List[dict]:
    """Each request alone, all its tokens in one step."""
    return [{"step": k, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for k, (rid, toks) in enumerate(reqs.items())]


def schedule_tail(reqs: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    """Each request alone: all but the last ``tail`` tokens in one step, then one token a step."""
    out, k = [], 0
    for rid, toks in reqs.items():
        head = max(1, len(toks) - tail)
        out.append({"step": k, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        k += 1
        for p in range(head, len(toks)):
            out.append({"step": k, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                        "end": [rid] if p == len(toks) - 1 else []})
            k += 1
        if head == len(toks):
            out[-1]["end"] = [rid]
    return out


def schedule_batches(reqs: Dict[str, List[int]], batch_size: int, decode: Sequence[int] = (3, 9, 1, 14, 6)) -> List[dict]:
    """Batches of ``batch_size`` requests, one batch after another.  In a batch every request brings a
    prompt (all but its last ``decode[i]`` tokens) in the first step, then one token a step; requests
    run out at different steps and leave the batch then."""
    ids = list(reqs)
    out, k = [], 0
    for b0 in range(0, len(ids), batch_size):
        batch = ids[b0:b0 + batch_size]
        heads = {rid: max(1, len(reqs[rid]) - decode[i % len(decode)]) for i, rid in enumerate(batch)}
        done_at = {rid: len(reqs[rid]) - heads[rid] for rid in batch}  # decode steps each request takes
        rec = {"step": k, "entries": [{"id": rid, "tokens": reqs[rid][:heads[rid]], "want": list(range(heads[rid]))}
                                      for rid in batch], "end": [rid for rid in batch if done_at[rid] == 0]}
        out.append(rec)
        k += 1
        for t in range(1, max(done_at.values()) + 1):
            live = [rid for rid in batch if done_at[rid] >= t]
            out.append({"step": k,
                        "entries": [{"id": rid, "tokens": [reqs[rid][heads[rid] + t - 1]], "want": [0]} for rid in live],
                        "end": [rid for rid in live if done_at[rid] == t]})
            k += 1
    return out


def schedule_staggered(reqs: Dict[str, List[int]], start_every: int = 2, decode: Sequence[int] = (6, 2, 11, 4),
                       chunks: Sequence = (None, 5, 19, 1)) -> List[dict]:
    """Requests join while others run: request i starts at step ``i * start_every``.  Its prompt (all but its last
    ``decode[i]`` tokens) comes whole (``chunks[i]`` None) or in pieces of ``chunks[i]`` tokens over consecutive
    steps, then one token a step.  So a step may hold single tokens of running requests beside whole or partial
    prompts of new ones; requests end at different steps, and later ones take the slots and pages they gave back."""
    ids = list(reqs)
    todo = {}
    for i, rid in enumerate(ids):
        toks = reqs[rid]
        head = max(1, len(toks) - decode[i % len(decode)])
        size = chunks[i % len(chunks)] or head
        pieces = [toks[a:min(a + size, head)] for a in range(0, head, size)] + [[t] for t in toks[head:]]
        todo[rid] = (i * start_every, pieces)
    out, k = [], 0
    while any(pieces for _, pieces in todo.values()):
        entries, end = [], []
        for rid in ids:
            start, pieces = todo[rid]
            if k < start or not pieces:
                continue
            piece = pieces.pop(0)
            entries.append({"id": rid, "tokens": piece, "want": list(range(len(piece)))})
            if not pieces:
                end.append(rid)
        out.append({"step": k, "entries": entries, "end": end})
        k += 1
    return out


def run_schedule(replayer, records: List[dict]) -> Dict[str, torch.Tensor]:
    """Replay ``records``; gather the logits of every wanted place per request, in position order."""
    got: Dict[str, Dict[int, torch.Tensor]] = {}
    fed: Dict[str, int] = {}
    for rec in records:
        logits = replayer.run(rec)
        row = 0
        for e in rec["entries"]:
            base = fed.get(e["id"], 0)
            for p in e.get("want", []):
                got.setdefault(e["id"], {})[base + p] = logits[row].float().cpu()
                row += 1
            fed[e["id"]] = base + len(e["tokens"])
        assert logits is None or row == logits.shape[0]
        replayer.cache.check_consistent()
    return {rid: torch.stack([rows[p] for p in sorted(rows)]) for rid, rows in got.items()}


def plain_logits(folder: str, reqs: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    cfg, w = plain.read_model(folder)
    return {rid: plain.forward(cfg, w, toks).float() for rid, toks in reqs.items()}


def plain_logits_on_gpu(folder: str, reqs: Dict[str, List[int]], last: int = 0) -> Dict[str, torch.Tensor]:
    """The plain implementation's float64 logits (of the last ``last`` places; 0: all) with its tensors on the GPU:
    the same functions as ``plain_logits``, plain torch, nothing of the engine, for sizes at which the CPU takes
    minutes."""
    cfg, w = plain.read_model(folder, device="cuda")
    out = {rid: plain.forward(cfg, w, toks, last=last).float().cpu() for rid, toks in reqs.items()}
    del w
    torch.cuda.empty_cache()
    return out


def lengths_reached(reqs: Dict[str, List[int]], records: List[dict]) -> Dict[str, List[int]]:
    """For every token of every request, the length its request had after the step that brought the token: what
    frequencies that follow a sequence's length look at."""
    out: Dict[str, List[int]] = {rid: [] for rid in reqs}
    for rec in records:
        for e in rec["entries"]:
            n = len(out[e["id"]]) + len(e["tokens"])
            out[e["id"]].extend([n] * len(e["tokens"]))
    assert all(len(out[rid]) == len(reqs[rid]) for rid in reqs)
    return out


def plain_logits_as_fed(folder: str, reqs: Dict[str, List[int]], records: List[dict]) -> Dict[str, torch.Tensor]:
    """The plain logits for a configuration whose result depends on the pieces a sequence was fed in."""
    cfg, w = plain.read_model(folder)
    lens = lengths_reached(reqs, records)
    return {rid: plain.forward(cfg, w, toks, seq_lens=lens[rid]).float() for rid, toks in reqs.items()}


def assert_close(got: torch.Tensor, want: torch.Tensor, rel: float, what: str) -> float:
    """max |got - want| <= rel * max |want|; returns the measured ratio."""
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    scale = float(want.abs().max())
    err = (got - want).abs()
    worst = float(err.max())
    if worst > rel * scale:
        idx = int(err.view(err.shape[0], -1).max(dim=1)[0].gt(rel * scale).nonzero()[0])
        raise AssertionError(
            f"{what}: max |diff| {worst:.3e} > {rel:g} x {scale:.3e}; first bad row (position) {idx} "
            f"of {err.shape[0]}, its max |diff| {float(err[idx].max()):.3e}")
    return worst / scale


# tolerances, relative to the largest logit of the request:
# 32-bit engine against the float64 plain implementation
REL_F32 = 2e-5
# bfloat16 engine (8 bits of mantissa, rounded after every layer op) against the same
REL_BF16 = 4e-2
