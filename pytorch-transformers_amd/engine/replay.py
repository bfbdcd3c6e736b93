"""Replaying a trace: requests named by ids, fed step by step through a model's step function.

One record of a trace is a dict ``{"step": k, "entries": [{"id", "tokens", "want"}...], "end": [ids]}``.
A step may hold any mix: whole prompts, pieces of prompts and single tokens of requests that are
already running; a request holds a cache slot from its first step until a record's ``end`` names it.  This is the whole of the program ``bin/trace_run`` apart
from reading lines and writing files, and what the tests drive in-process.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch


class Replayer:
    def __init__(self, model, max_tokens: int, max_slots: Optional[int] = None):
        self.model = model
        self.cache = model.new_cache(max_tokens, max_slots)
        self.slots: Dict[str, int] = {}

    def run(self, record: dict) -> Optional[torch.Tensor]:
        """Run one record; returns the wanted logits ``[wanted, vocab]`` (32-bit, on the device) or None."""
        entries = record.get("entries", [])
        logits = None
        if entries:
            ids = [e["id"] for e in entries]
            if len(set(ids)) != len(ids):
                raise ValueError(f"step {record.get('step')}: a request id appears twice: {ids}")
            for rid in ids:
                if rid not in self.slots:
                    self.slots[rid] = self.cache.alloc()
            want = [list(e.get("want", [])) for e in entries]
            out = self.model.step(self.cache, [self.slots[r] for r in ids], [e["tokens"] for e in entries], want)
            if out.shape[0] > 0:
                logits = out
        for rid in record.get("end", []):
            if rid in self.slots:
                self.cache.free(self.slots.pop(rid))
        return logits
