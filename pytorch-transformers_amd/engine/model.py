"""A causal language model put together from a ModelSpec, and its one step function.

The reference's forward pass takes a padded batch, a cache object, a mask and positions and returns
the logits of the last ``num_logits_to_keep`` places of every row
(src/transformers/models/falcon/modeling_falcon.py:1185-1254, :864-1011).  ``CausalLM.step`` takes,
for each sequence of a batch, its slot, the tokens it brings and the places whose logits are
wanted; it runs exactly those tokens from the cache, appends their keys and values, and returns the
wanted rows as 32-bit logits.  Whole prompts, single decoded tokens and any cut in between are the
same call.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import ctypes
import gc
import os
import weakref

import numpy as np
import torch

from .. import host, tuning
from ..cache.paged import PagedCache
from ..config.registry import AutoConfig, lookup
from ..parts.base import ResidualSum, StepContext, as_tensor
from ..weights.loader import load_weights
from ..weights.random_init import random_tensors
from .spec import ModelSpec
from .step import StepError, StepPlan, Want, plan_step

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def resolve_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be 'float32', 'bfloat16' or 'auto', got {dtype!r}") from None


def auto_dtype(config, folder: str) -> torch.dtype:
    """What ``dtype="auto"`` means (src/transformers/modeling_utils.py:3996-4058): the configuration's
    ``torch_dtype`` if it names one, else the type of the first floating-point tensor of the weight files.  The
    engine computes in bfloat16 or in 32-bit: 16-bit floats of the other kind run as bfloat16, wider ones in 32-bit."""
    from ..weights.loader import first_float_dtype

    named = getattr(config, "torch_dtype", None)
    if named is not None:
        name = str(named).replace("torch.", "")
        if name in ("bfloat16", "float16", "half"):
            return torch.bfloat16
        if name in ("float32", "float", "float64", "double"):
            return torch.float32
        raise ValueError(f"config.json names torch_dtype {named!r}, which the engine cannot compute in")
    found = first_float_dtype(folder)
    return torch.bfloat16 if found in (torch.bfloat16, torch.float16) else torch.float32


def _require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError(
            f"the engine runs on an AMD GPU through its HIP kernels and has no CPU path (device={device}, "
            f"torch.cuda.is_available()={torch.cuda.is_available()})")
    return device


GRAPH_LEN_STEP = 1024  # a decode graph serves contexts up to the next multiple of this ...
GRAPH_MEAN_STEP = 512  # ... whose mean is at most a multiple of this


def _len_bound(max_len: int) -> int:
    return (max_len + GRAPH_LEN_STEP - 1) // GRAPH_LEN_STEP * GRAPH_LEN_STEP


def mean_len_bound(total_len: int, n_seqs: int, len_bound: int) -> int:
    """The bucket of a step's mean context: its next multiple of ``GRAPH_MEAN_STEP``, at most ``len_bound``."""
    mean = -(-int(total_len) // max(1, int(n_seqs)))
    return min(len_bound, -(-mean // GRAPH_MEAN_STEP) * GRAPH_MEAN_STEP)


class _DecodeGraph:
    """One decode step of ``n`` sequences with contexts up to ``len_bound`` (``mean_bound`` on average),
    captured once and replayed.

    A decode step launches some ten kernels a layer; issued one by one from Python they cost more
    host time than the GPU needs to run them.  The captured graph reads everything that changes
    from step to step (token ids, positions, slots, page lists) from one device buffer, which a
    replay refreshes with a single copy from pinned host memory.  Launch shapes that depend on the
    context (how many key ranges the attention is split into) are sized for ``len_bound``; ranges
    past a sequence's end do no work.  A step with fewer than ``n`` sequences fills the spare rows with
    padding: token 0 as the first token of a sequence that lives in the cache's scratch slot and on its
    scratch page, which no sequence owns, so padding changes no sequence's keys, values or state, whatever
    the layers keep; the spare logits are dropped.  The first step of a graph's shape is launched directly
    (its result is the step's result) and the graph is captured after it, which runs nothing: no step's
    tokens go through the model twice.

    The cache owns its graphs and a graph refers to its cache weakly: with no cycle between them a cache
    that is dropped takes its graphs along at once.  A graph may not be destroyed while another one is
    being captured (the runtime refuses every such call during a capture, and the refusal, raised in a
    destructor, ends the process), and Python's collector of cycles runs when it pleases; for the same
    reason it is switched off while a capture lasts.
    """

    def __init__(self, model: "CausalLM", cache: PagedCache, n: int, len_bound: int, mean_bound: int = 0):
        self.model, self._cache, self.n, self.len_bound = model, weakref.ref(cache), n, len_bound
        self.mean_bound = mean_bound or len_bound
        self.width = len_bound // cache.page_size
        self.groups = cache.paged_groups()
        ar = np.arange(n, dtype=np.int32)
        # token_ids, token_seq, token_pos, cu_tokens, seq_start, seq_slot, logit_rows, then one table per group
        self.sizes = [n, n, n, n + 1, n, n, n] + [n * self.width] * len(self.groups)
        total = sum(self.sizes)
        self.host = torch.empty(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.offsets = np.concatenate([[0], np.cumsum(self.sizes)]).tolist()
        self._put(1, ar)
        self._put(3, np.arange(n + 1, dtype=np.int32))
        self._put(6, ar)
        self.dev = torch.zeros(total, dtype=torch.int32, device=model.device)
        self.copied = torch.cuda.Event()
        self.graph = None
        self.logits = None

    @property
    def cache(self) -> PagedCache:
        cache = self._cache()
        if cache is None:
            raise StepError("this decode graph's cache is gone")
        return cache

    def _put(self, i: int, arr) -> None:
        self.host_np[self.offsets[i]:self.offsets[i + 1]] = arr

    def _fill(self, plan: StepPlan) -> None:
        n, k = self.n, plan.n_seqs
        cache = self.cache
        pad = lambda a, fill=0: np.concatenate([a, np.full(n - k, fill, dtype=np.int32)]) if k < n else a
        self.copied.synchronize()  # the last copy out of the pinned buffer is done
        self._put(0, pad(plan.token_ids))
        self._put(2, pad(plan.token_pos))
        self._put(4, pad(np.asarray(plan.starts, dtype=np.int32)))
        self._put(5, pad(np.asarray(plan.slots, dtype=np.int32), cache.scratch_slot))
        for gi, g in enumerate(self.groups):
            t = np.zeros((n, self.width), dtype=np.int32)
            src = plan.block_tables[g]
            t[:k, :src.shape[1]] = src
            t[k:] = cache.scratch_page
            self._put(7 + gi, t.reshape(-1))
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()

    def _context(self):
        v = torch.split(self.dev, self.sizes)
        tables = {g: v[7 + i].view(self.n, self.width) for i, g in enumerate(self.groups)}
        ctx = StepContext(dtype=self.model.dtype, device=self.model.device, n_seqs=self.n, n_tokens=self.n,
                          token_seq=v[1], token_pos=v[2], cu_tokens=v[3], seq_start=v[4], seq_slot=v[5],
                          block_tables=tables, cache=self.cache, slots=[], new_tokens=[1] * self.n, starts=[],
                          is_decode=True, max_len=self.len_bound, mean_len=self.mean_bound)
        return ctx, v[0], v[6]

    def run(self, plan: StepPlan) -> torch.Tensor:
        """The step's logits, in a tensor of their own (the graph's output buffer is written again by the next
        replay)."""
        self._fill(plan)
        logits = self._launch()
        k = plan.n_seqs
        rows = plan.logit_rows
        if rows.shape[0] == k:  # one row per sequence, in order: the first k rows as they are
            return logits[:k].clone()
        if rows.shape[0] == 0:
            return logits[:0].clone()
        return logits.index_select(0, torch.from_numpy(rows.astype(np.int64)).to(logits.device))

    def run_last(self, n: int, slots_c, tokens_c, ids: Optional[torch.Tensor] = None,
                 own_logits: bool = True) -> torch.Tensor:
        """The common case, laid out by the host runtime straight into the pinned buffer: ``n`` sequences, one
        token each (C arrays), the logits of each.  ``ids``: the tokens as a tensor on the device, which takes
        the place of ``tokens_c`` there."""
        self.copied.synchronize()  # the last copy out of the pinned buffer is done
        lib = host.load()
        cache = self.cache
        rc = lib.ptah_decode_fill(cache.handle, n, slots_c, tokens_c, self.n, self.width, cache.scratch_slot,
                                  cache.scratch_page, self.host.data_ptr())
        if rc:
            raise StepError(host.last_error())
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        if ids is not None:
            self.dev[:n].copy_(ids)
        logits = self._launch()[:n]
        return logits.clone() if own_logits else logits

    def _launch(self) -> torch.Tensor:
        """Run the step that the device buffer now describes; returns the logits of all ``n`` rows (a buffer
        that the next call writes again)."""
        if self.graph is not None:
            self.graph.replay()
            return self.logits
        # the first step of this shape: launched directly, which also lets libraries set themselves up outside a
        # capture; its result is the step's result.  The capture that follows records launches and runs nothing.
        logits = self.model.forward_tokens(*self._context())
        graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()
        gc.disable()  # no finalizer of a dead cycle may call into the runtime while the capture lasts
        try:
            with torch.cuda.graph(graph):
                self.logits = self.model.forward_tokens(*self._context())  # a context of its own: nothing cached per step is shared
        finally:
            if collecting:
                gc.enable()
        self.graph = graph
        return logits


class CausalLM:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device):
        spec.validate()
        spec.check_sizes()
        self.spec = spec
        self.config = spec.config
        self.dtype = dtype
        self.device = torch.device(device)
        self.vocab_size = spec.head.vocab_size
        for part in spec.parts():
            part.load_all(tensors)
        for part in spec.parts():  # layouts that a part wants for its weights once they are there
            if hasattr(part, "after_load"):
                part.after_load()
        self._move_constants()
        self.generation_config = None
        #: the timed choices between kernels for this model's shapes (``tune``); active while this model steps
        self.tuning = tuning.TuningTable()
        #: run steps in which every sequence brings one token as replays of a captured HIP graph
        self.use_graphs = bool(spec.supports_graphs)
        #: ``layer_hook(i, x)`` is called after entry ``i`` of the run order with the residual stream
        #: ``[tokens, hidden]`` as a tensor (for dumps when a mismatch is being looked for); while it is set, steps
        #: are launched directly, never replayed from a captured graph
        self.layer_hook = None

    def _move_constants(self) -> None:
        seen = set()

        def walk(p):
            if id(p) in seen:
                return
            seen.add(id(p))
            if hasattr(p, "to"):
                p.to(self.device)
            for c in p.children():
                walk(c)

        for part in self.spec.parts():
            walk(part)

    # construction ----------------------------------------------------------
    @classmethod
    def from_pretrained(cls, folder: str, dtype="bfloat16", device="cuda:0", strict: bool = True,
                        tuning_table=None) -> "CausalLM":
        """``tuning_table``: choices between kernels that another process timed (``tune``), as the dict that
        ``tune`` returns or the path of a JSON file that holds it."""
        from ..config.generation import GenerationConfig

        device = _require_gpu(device)
        config = AutoConfig.from_pretrained(folder)
        dtype = auto_dtype(config, folder) if dtype == "auto" else resolve_dtype(dtype)
        _, builder = lookup(config.model_type)
        spec = builder(config)
        spec.validate()
        spec.check_sizes()  # a configuration that no kernel takes is refused before a weight is read
        tensors = load_weights(folder, spec.tensor_specs(), dtype, device, base_prefix=spec.base_prefix, strict=strict)
        model = cls(spec, tensors, dtype, device)
        model.generation_config = GenerationConfig.from_pretrained(folder, config)
        if tuning_table is not None:
            model.tune(table=tuning_table)
        return model

    @classmethod
    def from_config(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", std: Optional[float] = None,
                    noise: Optional[float] = None) -> "CausalLM":
        """Random weights drawn on the device; nothing is written to disk."""
        from ..config.generation import GenerationConfig

        device = _require_gpu(device)
        dtype = resolve_dtype(dtype)
        _, builder = lookup(config.model_type)
        spec = builder(config)
        spec.validate()
        spec.check_sizes()
        std = float(getattr(config, "initializer_range", 0.02) if std is None else std)
        specs = spec.tensor_specs()
        tensors = random_tensors(specs, seed, std, noise=noise, device=device, compute_dtype=dtype)
        for s in specs:
            if s.name not in tensors and s.tied_to is not None:
                tensors[s.name] = tensors[s.tied_to]
        model = cls(spec, tensors, dtype, device)
        model.generation_config = GenerationConfig.from_model_config(config)
        return model

    # timed choices ---------------------------------------------------------------
    @torch.no_grad()
    def tune(self, prompt_lens: Sequence[int] = (2048,), batches: Sequence[int] = (8, 64), table=None,
             contexts: Sequence = ()) -> dict:
        """Time, once, the choices between kernels that no rule decides, for prompts of ``prompt_lens`` tokens and
        decode steps of ``batches`` sequences, and keep them in this model's table (``self.tuning``) for every
        later step of this model; returns the table as plain data.  With ``contexts`` the decode steps are also run at these context lengths,
        each a number or a pair (longest, mean of the batch), over a cache that holds whatever it holds (only times
        are taken): that is where the cut of the decode attention is timed.  With ``table`` given (such data, or
        the path of a JSON file that holds it) nothing is timed: its choices are taken instead.
        Steps never time anything by themselves (unless PTA_TUNE=1 is set): untuned, they take the built-in
        choice, and logits are the same bits in every process."""
        tuning.activate(self.tuning)
        if table is not None:
            if isinstance(table, (str, os.PathLike)):
                import json

                with open(table) as f:
                    table = json.load(f)
            self.tuning.load(table)
            return self.tuning.to_dict()
        if self.dtype != torch.bfloat16:
            return self.tuning.to_dict()  # the 32-bit path has one kernel per operation
        graphs, self.use_graphs = self.use_graphs, False  # nothing can be timed inside a capture
        page = self.page_size
        pairs = sorted({(int(c), int(c)) if isinstance(c, int) else (int(c[0]), int(c[1])) for c in contexts})
        most = max([int(b) for b in batches] + [1])
        need = max([int(t) for t in prompt_lens] + [0]) + page * most + page
        need = max(need, most * ((max([c[0] for c in pairs] + [0]) + page) // page * page))
        cache = self.new_cache(need)
        timed: set = set()  # decode launches whose cuts have been timed in this call
        try:
            with tuning.live_tuning():
                for T in prompt_lens:
                    slot = cache.alloc()
                    self.step(cache, [slot], [[0] * int(T)], "last")
                    cache.free(slot)
                for b in (int(b) for b in batches):
                    # one token each: the shape of a decode step; then the same with tokens before it in every
                    # sequence, one sequence as long as the longest and the others such that the mean comes out
                    for longest, mean in [(1, 1)] + pairs:
                        rest = longest if b == 1 else max(1, min(longest, (mean * b - longest) // (b - 1)))
                        before = [longest - 1] + [rest - 1] * (b - 1)
                        slots = [cache.alloc() for _ in range(b)]
                        grow = [(s_, n_) for s_, n_ in zip(slots, before) if n_ > 0]
                        if grow:
                            cache.reserve([s_ for s_, _ in grow], [n_ for _, n_ in grow])
                            cache.commit([s_ for s_, _ in grow], [n_ for _, n_ in grow])
                        tuning.take_decode_keys()
                        self.step(cache, slots, [[0]] * b, "last")
                        if longest > 1 and graphs and os.environ.get("PTA_DECODE_TUNE", "1") != "0":
                            self._time_decode_cuts(cache, slots, timed)
                        for s_ in slots:
                            cache.free(s_)
            torch.cuda.synchronize()
        finally:
            self.use_graphs = graphs
            tuning.release_flush()
        return self.tuning.to_dict()

    def _time_decode_cuts(self, cache: PagedCache, slots: Sequence[int], timed: set, replays: int = 8,
                          rounds: int = 3) -> None:
        """For the decode launches of the step that was just run with timing on: capture the next step of these
        sequences once per candidate cut of the attention and keep the cut whose replays are fastest, if it beats
        the rule's by more than noise.  Whole steps are timed because a cut's time alone, after a flush of the
        caches, does not rank the cuts as a step does.  Nothing is committed: every replay writes the same
        position again."""
        keys = tuning.take_decode_keys()
        if not keys:
            return
        b = len(slots)
        plan = plan_step(cache, slots, [[0]] * b, "last", self.vocab_size)
        n_bucket = b if b <= 8 else (b + 7) // 8 * 8
        len_bound = _len_bound(plan.max_len)
        mean_bound = mean_len_bound(plan.total_len, b, len_bound)

        def step_ms() -> float:
            g = _DecodeGraph(self, cache, n_bucket, len_bound, mean_bound)
            g._fill(plan)
            g._launch()  # directly, then captured
            g._launch()
            best = float("inf")
            for _ in range(rounds):
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(replays):
                    g._launch()
                end.record()
                end.synchronize()
                best = min(best, start.elapsed_time(end) / replays)
            return best

        for key in keys:
            if key in timed:
                continue
            timed.add(key)
            cuts = tuning.decode_plan_candidates(key)
            times = []
            for cut in cuts:
                tuning.set_decode_plan(key, cut)
                times.append(step_ms())
            best = min(range(len(cuts)), key=lambda i: times[i])
            chosen = cuts[best] if times[best] < 0.985 * times[0] else None
            tuning.set_decode_plan(key, chosen)
            if os.environ.get("PTA_TUNE_VERBOSE"):
                print(f"[pta tune] decode attention {key}: " + " ".join(f"{c}:{t:.3f}" for c, t in zip(cuts, times))
                      + f" ms a step -> {chosen or cuts[0]}", flush=True)
        tuning.take_decode_keys()  # the steps above asked too

    @property
    def steps_ahead(self) -> bool:
        """Whether ``step`` can launch a step from tokens that are still on the device (a ``TokensAhead``) without
        waiting for them: where steps of one token per sequence are replays of a captured step."""
        return bool(self.use_graphs) and self.layer_hook is None

    # cache -------------------------------------------------------------------
    @property
    def page_size(self) -> int:
        """Tokens per cache page: a sequence's share of a cache is its length rounded up to this."""
        from ..cache.paged import PAGE_SIZE

        return PAGE_SIZE

    def new_cache(self, max_tokens: int, max_slots: Optional[int] = None) -> PagedCache:
        """A cache for at most ``max_tokens`` live tokens (each sequence's count rounded up to a page)."""
        return PagedCache(self.spec.cache_groups, max_tokens, self.dtype, self.device, max_slots=max_slots)

    # the step ------------------------------------------------------------------
    def make_context(self, plan: StepPlan, cache: PagedCache):
        """Upload a plan's arrays in one buffer and wrap the views."""
        n, M, R = plan.n_seqs, plan.n_tokens, int(plan.logit_rows.shape[0])
        names = list(plan.block_tables)
        dev = torch.from_numpy(plan.buffer).to(self.device)  # the host runtime laid the pieces out in one buffer
        views = torch.split(dev, plan.sizes)
        tables = {g: views[7 + i].view(plan.block_tables[g].shape) for i, g in enumerate(names)}
        ctx = StepContext(dtype=self.dtype, device=self.device, n_seqs=n, n_tokens=M, token_seq=views[1],
                          token_pos=views[2], cu_tokens=views[3], seq_start=views[4], seq_slot=views[5],
                          block_tables=tables, cache=cache, slots=plan.slots, new_tokens=plan.new_tokens,
                          starts=plan.starts, is_decode=plan.is_decode, max_len=plan.max_len,
                          mean_len=mean_len_bound(plan.total_len, n, _len_bound(plan.max_len)))
        return ctx, views[0], (views[6] if R else None)

    def forward_tokens(self, ctx: StepContext, token_ids: torch.Tensor, logit_rows: Optional[torch.Tensor]):
        """Embedding, the layers in their run order, final norm and head on the wanted rows."""
        x = self.spec.embedding.forward(token_ids)
        blocks = self.spec.blocks
        for i, call in enumerate(self.spec.order):
            block = blocks[call.block]
            if isinstance(x, ResidualSum) and not getattr(block, "accepts_sum", False):
                x = x.tensor()
            x = block.forward(x, ctx, call)
            if self.layer_hook is not None:
                self.layer_hook(i, as_tensor(x))  # a sum that is not formed yet is formed for the hook alone
        if logit_rows is None:
            return None
        norm = self.spec.final_norm
        if isinstance(x, ResidualSum) and norm is not None and hasattr(norm, "forward_sum"):
            h = norm.forward_sum(x, rows=logit_rows, want_x=False)[1]
        else:
            x = as_tensor(x)
            h = norm.forward(x, rows=logit_rows) if norm is not None else x.index_select(0, logit_rows.long())
        return self.spec.head.forward(h)

    def compute_transition_scores(self, output, prompt_lens, normalize_logits: bool = False):
        """``engine.generate.compute_transition_scores`` (the reference's method of the same name, without beams)."""
        from .generate import compute_transition_scores

        return compute_transition_scores(output, prompt_lens, normalize_logits)

    # decode steps as HIP graphs ---------------------------------------------------------
    def _graph_for(self, cache: PagedCache, plan: StepPlan) -> "_DecodeGraph":
        return self._graph_for_sizes(cache, plan.n_seqs, plan.max_len, plan.total_len)

    def _graph_for_sizes(self, cache: PagedCache, n: int, max_len: int, total_len: int) -> "_DecodeGraph":
        n_bucket = n if n <= 8 else (n + 7) // 8 * 8
        len_bound = _len_bound(max_len)
        mean_bound = mean_len_bound(total_len, n, len_bound)
        graphs = cache.__dict__.setdefault("_decode_graphs", {})
        key = (id(self), n_bucket, len_bound, mean_bound)
        g = graphs.get(key)
        if g is None:
            g = graphs[key] = _DecodeGraph(self, cache, n_bucket, len_bound, mean_bound)
        return g

    @torch.no_grad()
    def step(self, cache: PagedCache, slots: Sequence[int], tokens, want: Want = "last",
             own_logits: bool = True) -> torch.Tensor:
        """Run the given tokens of the given sequences; return logits ``[wanted places, vocab]`` in 32-bit.

        ``want`` is ``"last"``, ``"all"``, ``"none"`` or, per sequence, the places among its tokens
        of this step whose logits are asked for.  Rows come in the order of the sequences and of
        their places.

        ``tokens`` is a list of token lists, or a ``TokensAhead``: one token per sequence, chosen by the last step
        and still on the device, of which this step takes ``tokens.rows``; the step is then launched without a
        wait for them.  ``own_logits=False`` lets a step of one token per sequence return its logits in the buffer
        that the next such step writes again (for a caller that uses them at once).
        """
        from ..sampling.ahead import TokensAhead

        tuning.activate(self.tuning)
        graphs = self.use_graphs and self.layer_hook is None
        if isinstance(tokens, TokensAhead):
            if graphs and want == "last":
                return self._decode_last(cache, slots, None, ahead=tokens, own_logits=own_logits)
            seen = tokens.tolist()  # no captured step to launch them into: as any other tokens, once they are here
            tokens = [[seen[r]] for r in (tokens.rows if tokens.rows is not None else range(len(seen)))]
        if graphs and want == "last" and len(tokens) == len(slots) and all(len(t) == 1 for t in tokens):
            return self._decode_last(cache, slots, tokens, own_logits=own_logits)
        plan = plan_step(cache, slots, tokens, want, self.vocab_size)
        if graphs and plan.is_decode:
            logits = self._graph_for(cache, plan).run(plan)
            cache.commit(plan.slots, plan.new_tokens)
            return logits
        ctx, ids, rows = self.make_context(plan, cache)
        logits = self.forward_tokens(ctx, ids, rows)
        cache.commit(plan.slots, plan.new_tokens)
        if logits is None:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        return logits

    def _decode_last(self, cache: PagedCache, slots: Sequence[int], tokens, ahead=None,
                     own_logits: bool = True) -> torch.Tensor:
        """One token per sequence, the logits of each, as a replay of a captured step: the host runtime checks
        the step, reserves pages and writes the step's integers straight into the buffer that is copied to
        the device.  ``ahead``: the tokens are not ``tokens`` but rows of a tensor on the device, which are copied
        into the step's buffer there."""
        from ..cache.paged import CacheError, CacheFull

        n = len(slots)
        if n == 0:
            raise StepError("a step needs at least one sequence")
        if ahead is not None and n != (len(ahead.rows) if ahead.rows is not None else len(ahead)):
            raise StepError(f"{n} sequences, but tokens ahead for "
                            f"{len(ahead.rows) if ahead.rows is not None else len(ahead)}")
        lib = host.load()
        slots_c = (ctypes.c_int * n)(*[int(s) for s in slots])
        tokens_c = (ctypes.c_longlong * n)() if ahead is not None else (ctypes.c_longlong * n)(*[int(t[0]) for t in tokens])
        longest, total = ctypes.c_int(0), ctypes.c_longlong(0)
        rc = lib.ptah_decode_prepare(cache.handle, n, slots_c, tokens_c, self.vocab_size, ctypes.byref(longest),
                                     ctypes.byref(total))
        if rc:
            raise {host.ERR_STEP: StepError, host.ERR_FULL: CacheFull}.get(rc, CacheError)(host.last_error())
        logits = self._graph_for_sizes(cache, n, longest.value, total.value).run_last(
            n, slots_c, tokens_c, ids=None if ahead is None else ahead.for_step(), own_logits=own_logits)
        lib.ptah_commit_ones(cache.handle, n, slots_c)
        return logits

    # generation (see engine.generate) -----------------------------------------------
    def generate(self, prompts=None, generation_config=None, *, input_ids=None, **kwargs):
        """``engine.generate.generate`` for this model; ``input_ids=`` (with ``attention_mask=``) is the reference's
        spelling of tensor prompts, so ``model.generate(**tokenizer(texts, return_tensors="pt", padding=True))`` works."""
        from .generate import generate

        if prompts is None:
            prompts = input_ids
        elif input_ids is not None:
            raise ValueError("prompts were given twice: positionally and as input_ids")
        if prompts is None:
            raise ValueError("generate needs prompts: lists of token ids, or input_ids as a tensor")
        return generate(self, prompts, generation_config, **kwargs)
