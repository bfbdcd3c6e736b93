"""Choices between ways to the same result that are timed rather than ruled, and the table that keeps them.

Some choices have no rule that holds across shapes: how many ranges of K a pair launch is cut into, up to how many
rows the decode batch kernel beats the vendor library, in which pieces along M the library's product runs, whether
two matrices of one input run as one product, whether K is cut into a batch, and how a decode step's attention
launch is cut (for which there is a fitted model of the launch's time, below, that the timing may overrule).  Each
has a built-in default and an entry per shape in a ``TuningTable`` that overrides it.  A table is filled only while
timing is switched on: inside ``live_tuning()`` (``CausalLM.tune`` runs steps of given sizes in it), or in every
step with PTA_TUNE=1 in the environment.  With timing off (the default) a step allocates nothing for measurements
and times nothing, and its results depend on weights, tokens, schedule and table alone: two processes give the
same bits.  ``TuningTable.to_dict`` / ``load`` carry a table from one process to another.

``ops`` holds the kernel faces and asks here; this module calls the faces back when it times them.  The names of
this module are also reachable as attributes of ``ops``.
"""
from __future__ import annotations

import functools
import os
from typing import Optional

import torch

from . import ops


class TuningTable:
    """The choices that were timed rather than ruled, by shape.  A model owns one (``CausalLM.tuning``); callers of
    the kernel faces that bring none share ``DEFAULT``.  The table whose choices hold is the active one
    (``activate``): a model activates its own at the start of every step, so two models in one process neither see
    nor overwrite each other's choices.  The ranges of K of pair launches are also kept inside the kernel library,
    by shape; ``activate`` takes the old table's out of it and puts the new one's in."""

    FIELDS = ("pair_parts", "pair_stationary", "splitk_rows", "mm_plans", "mm_joined", "mm_ksplit", "decode_plans")

    def __init__(self, data: Optional[dict] = None):
        self.pair_parts: dict = {}  # (shape of w1, shape of w2) -> (ranges, ranges, row tiles per wave) in use
        # (shape of w1, shape of w2) -> per class of rows the (ranges, ranges) of the launch with stationary
        # activations, (0, 0) where the staged kernel stays
        self.pair_stationary: dict = {}
        self.splitk_rows: dict = {}  # ((N, K), ...) -> rows up to which the batch kernel beats the library's product
        self.mm_times: dict = {}  # (N, K) -> {rows: microseconds}; measurements, not part of the table as data
        self.mm_plans: dict = {}  # (N, K, M bucket) -> [rows, ...]
        self.mm_costs: dict = {}  # (N, K, M bucket) -> microseconds of that plan, as measured piece by piece
        self.mm_joined: dict = {}  # (N1, N2, K, M bucket) -> whether one product with both matrices beats the two
        self.mm_ksplit: dict = {}  # (N, K, M bucket) -> ranges of K (1: the plain product)
        self.decode_plans: dict = {}  # (batch, heads, KV heads, head size, longest, mean) as counted -> a timed cut
        if data:
            self.load(data)

    def to_dict(self) -> dict:
        """The table as plain data (JSON-able): loaded in another process, that process makes the same choices,
        hence the same bits."""
        key = lambda t: ",".join("x".join(str(int(v)) for v in (p if isinstance(p, tuple) else (p,))) for p in t)
        return {
            "pair_parts": {key(k): list(v) for k, v in self.pair_parts.items()},  # ranges, ranges, row tiles per wave
            "pair_stationary": {key(k): [list(c) for c in v] for k, v in self.pair_stationary.items()},  # per class of rows
            "splitk_rows": {key(k): int(v) for k, v in self.splitk_rows.items()},
            "mm_plans": {key(k): list(v) for k, v in self.mm_plans.items()},
            "mm_joined": {key(k): bool(v) for k, v in self.mm_joined.items()},
            "mm_ksplit": {key(k): int(v) for k, v in self.mm_ksplit.items()},
            "decode_plans": {key(k): list(v) for k, v in self.decode_plans.items()},  # tiles, keys per workgroup, waves
        }

    def load(self, data: dict) -> None:
        """Take the choices of a table that ``to_dict`` made (entries for other shapes stay as they are).  The table
        becomes the active one, so that what it says about pair launches is checked by the kernel library now."""
        unknown = sorted(set(data) - set(self.FIELDS))
        if unknown:
            raise ValueError(f"a tuning table has the sections {list(self.FIELDS)}; this one also holds {unknown}")
        activate(self)
        shapes = lambda k: tuple(tuple(int(v) for v in p.split("x")) for p in k.split(","))
        flat = lambda k: tuple(int(p) for p in k.split(","))
        for k, v in data.get("pair_parts", {}).items():
            s1, s2 = shapes(k)
            cut = (int(v[0]), int(v[1]), int(v[2]) if len(v) > 2 else 1)
            _unfix_pair(s1, s2)
            _fix_pair(s1, s2, cut)
            self.pair_parts[(s1, s2)] = cut
        for k, v in data.get("pair_stationary", {}).items():
            s1, s2 = shapes(k)
            cuts = tuple((int(c[0]), int(c[1])) for c in v)
            _fix_stationary(s1, s2, cuts)
            self.pair_stationary[(s1, s2)] = cuts
        for k, v in data.get("splitk_rows", {}).items():
            self.splitk_rows[shapes(k)] = int(v)
        for k, v in data.get("mm_plans", {}).items():
            self.mm_plans[flat(k)] = [int(r) for r in v]
        for k, v in data.get("mm_joined", {}).items():
            self.mm_joined[flat(k)] = bool(v)
        for k, v in data.get("mm_ksplit", {}).items():
            self.mm_ksplit[flat(k)] = int(v)
        for k, v in data.get("decode_plans", {}).items():
            self.decode_plans[flat(k)] = tuple(int(p) for p in v)

    def clear(self) -> None:
        """Back to the built-in defaults for every shape."""
        if self is _active:
            _release(self)
        for d in (self.pair_stationary, self.pair_parts, self.splitk_rows, self.mm_plans, self.mm_costs, self.mm_times,
                  self.mm_joined, self.mm_ksplit, self.decode_plans):
            d.clear()


def _unfix_pair(s1, s2) -> None:
    ops.load_library().pta_gemm_splitk_pair_fix(int(s1[0]), int(s1[1]), int(s2[0]), int(s2[1]), 0, 0, 1)


def _fix_pair(s1, s2, cut) -> None:
    """Fix (ranges, ranges, row tiles per wave) for a pair of shapes in the kernel library, unless it is the rule's
    own choice (nothing is fixed for the shapes when this is called)."""
    a, b, rt = cut
    rule = ops.gemm_splitk_pair_parts(s1[0], s1[1], s2[0], s2[1])
    if (a, b, rt) != tuple(rule) + (1,) and ops.load_library().pta_gemm_splitk_pair_fix(
            int(s1[0]), int(s1[1]), int(s2[0]), int(s2[1]), int(a), int(b), int(rt)):
        raise ops.KernelError(f"tuning table: {a} and {b} ranges of K with {rt} row tiles are not valid for the pair "
                              f"{tuple(s1)}, {tuple(s2)}")


def _fix_stationary(s1, s2, cuts) -> None:
    lib = ops.load_library()
    for cls, c in enumerate(cuts):
        if lib.pta_gemm_splitk_pair_fix_stationary(int(s1[0]), int(s1[1]), int(s2[0]), int(s2[1]), cls, int(c[0]), int(c[1])):
            raise ops.KernelError(f"tuning table: {list(c)} is not valid for the pair {tuple(s1)}, {tuple(s2)} with "
                                  "stationary activations")


def _release(table: "TuningTable") -> None:
    """Take what ``table`` fixed for pair launches out of the kernel library."""
    if not table.pair_parts and not table.pair_stationary:
        return
    lib = ops.load_library()
    for (s1, s2) in table.pair_parts:
        _unfix_pair(s1, s2)
    for (s1, s2) in table.pair_stationary:
        lib.pta_gemm_splitk_pair_fix_stationary(int(s1[0]), int(s1[1]), int(s2[0]), int(s2[1]), -1, 0, 0)


def _apply(table: "TuningTable") -> None:
    for (s1, s2), cut in table.pair_parts.items():
        _fix_pair(s1, s2, cut)
    for (s1, s2), cuts in table.pair_stationary.items():
        _fix_stationary(s1, s2, cuts)


DEFAULT = TuningTable()  # of whoever calls the kernel faces without a table of their own
_active = DEFAULT


def active() -> TuningTable:
    return _active


def activate(table: Optional[TuningTable]) -> TuningTable:
    """Make ``table`` (None: ``DEFAULT``) the one whose choices hold, and the one that timing fills."""
    global _active
    table = DEFAULT if table is None else table
    if table is not _active:
        _release(_active)
        _active = table
        _apply(table)
    return table


def tuning_table() -> dict:
    """The active table as plain data."""
    return _active.to_dict()


def clear_tuning() -> None:
    """The active table back to the built-in defaults for every shape."""
    _active.clear()


def load_tuning(table: dict) -> None:
    """Take a table's choices into the active one."""
    _active.load(table)


# ---- the cut of a decode step's attention launch --------------------------------------------------------
@functools.lru_cache(maxsize=None)
def _decode_plan(n: int, n_heads: int, n_kv_heads: int, head_dim: int, bound: int, mean: int, most_tiles: int):
    """The cheapest cut of a decode launch of ``n`` sequences of up to ``bound`` keys, ``mean`` on average,
    by a model of its time.

    A wave holds ``t`` groups of sixteen heads of one KV head and walks ``size`` keys in blocks of 32.  In
    microseconds, fitted to launches with cold caches at three head shapes (71 heads on 1 KV head of 64; 32 on
    8 of 128; 128 on 8 of 64), 1 to 64 sequences of 1,100 to 8,192 keys, every cut (the model's choice is
    within a tenth of the best measured cut nearly everywhere, and mostly equal to it):

    - a wave takes 0.22 + 0.21 t + 0.15 (head_dim / 64 - 1) per block, and waves beyond what the chip
      holds at once (1,024 SIMDs, as many waves each as 512 registers allow) wait for a whole round;
    - the keys and values stream at 5.1 TB/s, and again at 7.2 TB/s for every further wave that shares
      a KV head;
    - the launch takes the 4.2-norm of those two times (the larger one, and more where they are close);
    - ranges cost 2.2 + 0.1 per range, and their partial sums (32-bit, written and read) move at 3.5 TB/s.

    The longest context of a step that is sized for ``bound`` lies in its last 1,024 and the mean in the 512
    below ``mean``, so the longest wave's time is taken at ``bound - 512`` keys and the traffic at
    ``mean - 256`` keys a sequence."""
    groups = (n_heads // n_kv_heads + 15) // 16
    dt = head_dim / 16.0
    keys = bound - 512
    mean_keys = min(keys, mean - 256)
    kv_mb = n * mean_keys * n_kv_heads * head_dim * 4 / 1e6
    best = None
    for t in range(1, most_tiles + 1):
        if ops.ATTN_FORCE_TILES and t != min(ops.ATTN_FORCE_TILES, most_tiles):
            continue
        sharing = (groups + t - 1) // t
        resident = 1024 * max(1, int(512 // ((38 + 11.5 * dt) + (26 + 8 * dt) * t)))
        block_us = 0.22 + 0.21 * t + 0.15 * (head_dim / 64.0 - 1.0)
        size = min(ops.ATTN_SPLIT_KEYS, ops.ATTN_FORCE_SPLIT) if ops.ATTN_FORCE_SPLIT else ops.ATTN_SPLIT_KEYS
        while True:
            whole = size >= bound
            if (bound + size - 1) // size <= 1024 and n * ((bound + size - 1) // size) <= 65535 and (not ops.ATTN_FORCE_SPLIT or size == ops.ATTN_FORCE_SPLIT or
                                                       (whole and size < ops.ATTN_FORCE_SPLIT)):
                ranges = (mean_keys + size - 1) // size
                waves = n * n_kv_heads * sharing * ranges
                wave_us = min(size, keys) / 32 * block_us * ((waves + resident - 1) // resident)
                stream_us = kv_mb / 5.1 + kv_mb * (sharing - 1) / 7.2
                part_us = 0.0 if whole else 2.2 + 0.1 * ranges + n * n_heads * ranges * head_dim * 8 / 1e6 / 3.5
                cost = (wave_us ** 4.2 + stream_us ** 4.2) ** (1 / 4.2) + part_us
                if best is None or cost < best[0]:
                    best = (cost, t, size)
            if whole:
                break
            size *= 2
    if best is None:
        raise ops.KernelError(f"no cut of a decode launch over {bound} keys with PTA_ATTN_SPLIT={ops.ATTN_FORCE_SPLIT}")
    return best[1], best[2]




def decode_key(n_seqs: int, n_heads: int, n_kv_heads: int, head_dim: int, max_len: int, mean_len: int):
    n = 1
    while n < n_seqs:
        n *= 2
    bound = (max_len + 1023) // 1024 * 1024
    mean = min(bound, (mean_len + 511) // 512 * 512) if mean_len > 0 else bound
    return (n, int(n_heads), int(n_kv_heads), int(head_dim), bound, mean)


def decode_plan(n_seqs: int, n_heads: int, n_kv_heads: int, head_dim: int, max_len: int, mean_len: int = 0):
    """How a decode launch is cut: (column tiles per wave, keys per workgroup, waves per workgroup); a size that
    covers the context means one workgroup per sequence and head group, which writes the result itself.  The
    waves of a workgroup take its keys block by block in turn and merge in LDS; ``SHARED_KEYS`` in their place
    means a wave per tile of heads, all on the same keys (``_shared_keys_rule``).

    The batch counts by its next power of two, the longest context by its next multiple of 1,024 and the
    mean context (``mean_len``; 0: as the longest) by its next multiple of 512, so that a captured step,
    which is sized for a padded batch and such bounds, is cut exactly as the same step run directly.
    A cut that was fixed for these counts (``set_decode_plan``; ``CausalLM.tune`` times whole steps with the cuts
    of ``decode_plan_candidates``) goes before the rule, which has one wave per workgroup or shared keys."""
    key = decode_key(n_seqs, n_heads, n_kv_heads, head_dim, max_len, mean_len)
    kept = _active.decode_plans.get(key)
    if kept is not None:
        return kept
    n, _, _, _, bound, mean = key
    shared = _shared_keys_rule(n, n_heads, n_kv_heads, head_dim, bound, mean)
    if shared is not None:
        return shared
    groups = (n_heads // n_kv_heads + 15) // 16
    most = min(groups, int(ops.load_library().pta_attn_decode_max_tiles(head_dim)))
    return _decode_plan(n, n_heads, n_kv_heads, head_dim, bound, mean, most) + (1,)


def _shared_keys_rule(n: int, n_heads: int, n_kv_heads: int, head_dim: int, bound: int, mean: int):
    """The cut with keys shared through LDS where it is built (many heads on a KV head) and the launch walks keys
    enough to fill the chip with such workgroups, else None.  Measured with 71 heads on one KV head of 64, launch
    and merge after a flush of the caches, against the best cut of one-wave workgroups: 8 sequences of 1,100 keys
    11.4 against 9.8 us; 32 of 1,100 10.3 against 15.4; 64 of 2,100 14.8 against 26.0; 8 of 16,384 19.8 against
    24.8; 32 of 16,384 45.6 against 49.8.  Ranges of 256 keys up to 100 k keys in all, 512 up to 300 k, then 1,024."""
    if ops.ATTN_FORCE_SPLIT or ops.ATTN_FORCE_TILES or not ops.attn_decode_shared_ok(head_dim, n_heads // n_kv_heads):
        return None
    keys = n * n_kv_heads * mean
    if keys < 20_000:
        return None
    size = 256 if keys <= 100_000 else 512 if keys <= 300_000 else 1024
    while size < bound and ((bound + size - 1) // size > 1024 or n * ((bound + size - 1) // size) > 65535):
        size *= 2  # the launch's limits: ranges of a sequence, and sequences x ranges
    return (1, min(size, bound), ops.SHARED_KEYS)


_decode_keys_seen: set = set()  # what decode launches asked ``decode_plan`` for while timing was on


def note_decode_launch(n_seqs: int, n_heads: int, n_kv_heads: int, head_dim: int, max_len: int, mean_len: int = 0) -> None:
    """While timing is on: remember that a decode launch of this shape ran, for ``CausalLM.tune`` to time its cuts."""
    if may_time():
        _decode_keys_seen.add(decode_key(n_seqs, n_heads, n_kv_heads, head_dim, max_len, mean_len))


def take_decode_keys() -> list:
    """The (batch, head shape, context) counts of the decode launches since the last call, while timing was on."""
    keys = sorted(_decode_keys_seen)
    _decode_keys_seen.clear()
    return keys


def decode_plan_candidates(key) -> list:
    """Cuts of the decode launch that ``key`` counts, the rule's first: the one-wave rule's neighbours,
    workgroups of four and eight waves over the whole context and over ranges of 512 and 1,024 keys, and, where
    they are built, workgroups that share their keys over ranges of 256 to 1,024 keys and the whole context.  A workgroup of several waves needs no second launch when it walks the whole context, but all its keys
    pass through one compute unit; which wins depends on how many sequences and KV heads there are to fill the
    chip.  Timed alone after a flush of the caches, these cuts rank differently than inside a step (the rule's
    cut at 64 sequences, 8 KV heads of 64 and 1,100 keys: 42 us alone, 31 us in a step, where a cut with four
    waves takes 34 us both times), so the caller times whole steps with each (``CausalLM.tune``)."""
    n, nh, nkv, d, bound, mean = key
    lib = ops.load_library()
    groups = (nh // nkv + 15) // 16
    most = min(groups, int(lib.pta_attn_decode_max_tiles(d)))
    rule = _decode_plan(n, nh, nkv, d, bound, mean, most) + (1,)
    shared = _shared_keys_rule(n, nh, nkv, d, bound, mean)
    cuts = [rule] if shared is None else [shared, rule]
    want = [(rule[0], rule[1] * 2, 1), (rule[0], rule[1] // 2, 1), (max(1, rule[0] - 1), rule[1], 1),
            (min(most, rule[0] + 1), rule[1], 1)]
    want += [(t, size, w) for t in (1, min(2, most)) for w in (4, 8) for size in (bound, 1024, 512)]
    for t, size, w in want:
        size = min(size, bound)
        splits = (bound + size - 1) // size
        if (size < ops.ATTN_SPLIT_KEYS or size % 64 or size // w < 64 or splits > 1024 or n * splits > 65535 or (t, size, w) in cuts
                or not lib.pta_attn_decode_waves_ok(d, t, w)):
            continue
        cuts.append((t, size, w))
    if ops.attn_decode_shared_ok(d, nh // nkv):
        for size in (256, 512, 1024, bound):
            cut = (1, min(size, bound), ops.SHARED_KEYS)
            splits = (bound + cut[1] - 1) // cut[1]
            if cut not in cuts and splits <= 1024 and n * splits <= 65535:
                cuts.append(cut)
    return cuts


def set_decode_plan(key, cut=None) -> None:
    """Fix the cut of the decode launches that ``key`` counts (None: back to the rule)."""
    if cut is None:
        _active.decode_plans.pop(tuple(key), None)
    else:
        _active.decode_plans[tuple(key)] = tuple(int(v) for v in cut)


# ---- when choices are timed -----------------------------------------------------------------------------
TUNE_LIVE = os.environ.get("PTA_TUNE", "0") == "1"


class live_tuning:
    """Context in which choices that have no entry in the tuning table yet are timed at first use."""

    def __enter__(self):
        global TUNE_LIVE
        self._old, TUNE_LIVE = TUNE_LIVE, True
        return self

    def __exit__(self, *exc):
        global TUNE_LIVE
        TUNE_LIVE = self._old
        return False


def may_time() -> bool:
    return TUNE_LIVE and not torch.cuda.is_current_stream_capturing()


SKINNY_MAX_ROWS = 64
# rows up to which the decode batch kernel (x shared through LDS, K split over workgroups) stands in for the
# vendor library's product, whose choices for 65 to 128 rows leave most of the chip idle (K = 4,544 with N =
# 4,672 and 18,176 in one product of 128 rows: 151 us, 1.4 TB/s of weights)
SPLITK_MAX_ROWS = int(os.environ.get("PTA_SPLITK_MAX_ROWS", "256"))
SPLITK_MARGIN = float(os.environ.get("PTA_SPLITK_MARGIN", "0.95"))
SPLITK_SURE_ROWS = 128  # up to here the kernel won at every shape measured; beyond, by the weight's own timing


_flush = None  # half a gigabyte that is read between timed runs; held only while timing is on (``release_flush``)


def release_flush() -> None:
    global _flush
    _flush = None


def time_ways_cold(ways, device, rounds: int = 3):
    """Milliseconds of each of ``ways`` (callables), the fastest of ``rounds`` runs each, taken in turn; before
    every run half a gigabyte is read, so that the weights come from memory as they do in a model (timed back
    to back, a product finds its matrix in the memory-side cache and every way looks alike).  Read, not
    written: after half a gigabyte of writes the caches are full of lines that must go back to memory before
    anything else comes in, which no step of a model leaves behind, and a kernel that streams from memory then
    measures at little more than half its speed (decode attention over 144 MB of keys and values: 55 us after
    writes, 31 us in a step)."""
    global _flush
    if _flush is None or _flush.device != device:
        _flush = torch.zeros(128 * 1024 * 1024, dtype=torch.float32, device=device)
    flush = _flush
    best = [float("inf")] * len(ways)
    for run in ways:  # plans are made and the library set up before anything is timed
        run()
    for _ in range(rounds):
        for i, run in enumerate(ways):
            flush.sum()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            run()
            end.record()
            end.synchronize()
            best[i] = min(best[i], start.elapsed_time(end))
    return best


def splitk_row_limit(*ws: torch.Tensor) -> int:
    """Rows up to which the decode batch kernel is the faster way to the product with ``w`` (or, for two weights, to
    the two products of a pair launch).  Up to 128 rows it always was (one chunk of rows per workgroup); with two
    chunks it depends on how well the library does at the shape (at 256 rows it wins with K = 4,544, 9.5 against
    11.4 ms a step of 32 layers, and loses with K = 4,096, 22.1 against 20.2 ms of 60 layers), so both are timed once
    per shape at 192 and 256 rows, when timing is on; without an entry the kernel stops at 128 rows."""
    if SPLITK_MAX_ROWS <= SPLITK_SURE_ROWS:
        return SPLITK_MAX_ROWS
    key = tuple(tuple(w.shape) for w in ws)
    limit = _active.splitk_rows.get(key)
    if limit is None:
        if not may_time():
            return SPLITK_SURE_ROWS
        dev = ws[0].device
        xs = [torch.randn((256, w.shape[1]), dtype=torch.float32, device=dev).to(torch.bfloat16) for w in ws]
        outs = [torch.empty((256, w.shape[0]), dtype=torch.bfloat16, device=dev) for w in ws]
        limit = SPLITK_SURE_ROWS
        for rows in (192, 256):
            if rows > SPLITK_MAX_ROWS:
                break
            xr = [x[:rows] for x in xs]

            def kernel():
                if len(ws) == 1:
                    ops.gemm_splitk_bf16(xr[0], ws[0])
                else:
                    ops.gemm_splitk_pair_bf16(xr[0], ws[0], xr[1], ws[1])

            def library():
                for x, w, out in zip(xr, ws, outs):
                    torch.mm(x, w.t(), out=out[:rows])

            best = time_ways_cold((kernel, library), dev)
            if best[0] < SPLITK_MARGIN * best[1]:
                limit = rows
            else:
                break
        _active.splitk_rows[key] = limit
    return limit


def splitk_rows_ok(x: torch.Tensor, *ws: torch.Tensor) -> bool:
    return x.shape[0] <= SPLITK_SURE_ROWS or x.shape[0] <= splitk_row_limit(*ws)


# ---- the vendor library's product for many rows, cut along M where that is faster -----------------------
# The library picks a kernel per (M, N, K) from a table, and on this hardware its choices are uneven in M:
# with K = 4,544 and N = 18,176, 2,048 rows take longer than 2,304, and 4,096 rows of the product with the
# transposed shape almost as long as 8,192.  So, when timing is on, the product is timed once per weight shape at
# a ladder of row counts, and a product of M rows then runs as the cheapest sequence of those pieces (each written
# straight into its rows of the result); without an entry it runs whole.  PTA_MM_CHUNKS=0 switches this off.
MM_LADDER = (256, 512, 768, 1024, 1536, 2048, 3072, 4096, 6144, 8192)
MM_CHUNKS = os.environ.get("PTA_MM_CHUNKS", "1") != "0"
MM_JOIN = os.environ.get("PTA_MM_JOIN", "1") != "0"  # one product for two matrices of one input where it is faster


def mm_measure(x: torch.Tensor, w: torch.Tensor, rows: int, out: torch.Tensor) -> float:
    """Microseconds of ``x[:rows] @ w.T``: the fastest of five runs, each timed on its own (a mean over two runs
    right after the library's set-up misjudged products by a tenth, enough to choose the slower plan)."""
    torch.mm(x[:rows], w.t(), out=out[:rows])  # the library's first call of a shape sets it up
    best = float("inf")
    for _ in range(5):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        torch.mm(x[:rows], w.t(), out=out[:rows])
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e3)
    return best


def mm_plan(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor):
    M, (N, K) = x.shape[0], w.shape
    bucket = (M + 63) // 64  # row counts within 64 of each other share a plan: one timing of the whole product
    plan = _active.mm_plans.get((N, K, bucket))
    if plan is not None:
        return plan[:-1] + [M - sum(plan[:-1])]
    if not may_time():
        return [M]
    times = _active.mm_times.setdefault((N, K), {})
    for rows in MM_LADDER:
        if rows <= M and rows not in times:
            times[rows] = mm_measure(x, w, rows, out)
    whole = M <= MM_LADDER[-1]  # beyond the ladder the product always runs in pieces: timing it whole costs too much
    if whole and M not in times:
        times[M] = mm_measure(x, w, M, out)  # the product as it is
    # cheapest way to cover M rows with pieces of the ladder; what is left over rides on the last piece
    units, rest = divmod(M, 256)
    best = [(0.0, [])] + [None] * units
    for u in range(1, units + 1):
        for rows in MM_LADDER:
            k = rows // 256
            if k <= u and rows in times and best[u - k] is not None:
                cand = best[u - k][0] + times[rows]
                if best[u] is None or cand < best[u][0]:
                    best[u] = (cand, best[u - k][1] + [rows])
    cost, pieces = best[units]
    if rest:
        pieces = pieces[:-1] + [pieces[-1] + rest]
        cost *= M / (M - rest)
    plan = pieces if not whole or (len(pieces) > 1 and cost < 0.97 * times[M]) else [M]
    _active.mm_plans[(N, K, bucket)] = plan
    _active.mm_costs[(N, K, bucket)] = cost if plan is pieces else times[M]
    return plan


def joined_mm_pays(x: torch.Tensor, joined: torch.Tensor, n_first: int) -> bool:
    """Whether ``x @ joined.T`` in one library product beats the products with its first ``n_first`` rows and
    with the rest on their own.  The library's kernel choice decides, so both ways are timed once per shape when
    timing is on (2,048 rows, K = 4,544, N = 4,672 + 18,176: 308 us against 87 + 286; K = 4,096, N = 6,144 + 16,384:
    311 against 80 + 179); without an entry the two stay apart."""
    M, (N, K) = x.shape[0], joined.shape
    if not MM_JOIN or not MM_CHUNKS or M < 512:
        return False
    bucket = (M + 63) // 64
    key = (n_first, N - n_first, K, bucket)
    if key not in _active.mm_joined:
        if not may_time():
            return False
        first, rest = joined[:n_first], joined[n_first:]
        ways = (lambda: ops.library_mm(x, joined), lambda: (ops.library_mm(x, first), ops.library_mm(x, rest)))
        best = [float("inf"), float("inf")]
        for run in ways:  # plans are made and the library set up before anything is timed
            run()
        for _ in range(4):  # the two ways in turn, each run timed on its own; the fastest of each counts
            for i, run in enumerate(ways):
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                run()
                end.record()
                end.synchronize()
                best[i] = min(best[i], start.elapsed_time(end))
        _active.mm_joined[key] = best[0] < 0.98 * best[1]
    return _active.mm_joined[key]


# Ranges of K for the pairs of a shape: the kernel library's rule gives a choice; when timing is on, its neighbours
# are timed once per shape, at 64 rows, with cold caches, and one that is at least 3 % faster is kept for every
# later launch (PTA_PAIR_TUNE=0 switches this off).
PAIR_TUNE = os.environ.get("PTA_PAIR_TUNE", "1") != "0"
PAIR_TUNE_MARGIN = 0.97
PAIR_TUNE_ROWS = int(os.environ.get("PTA_PAIR_TUNE_ROWS", "64"))  # rows of the timed launches (17 to 128)


def tune_pair_parts(w1: torch.Tensor, w2: torch.Tensor) -> None:
    """Once per pair of shapes, while timing is on: time the pair launch with the rule's ranges of K, with their
    neighbours, and with workgroups of 128 rows of W (which load the activations half as often, have half as many
    workgroups and so want more ranges), at 64 rows with cold caches; keep the fastest in the kernel library if it
    beats the rule's by the margin and is no slower than the rule's at 24 rows (where the tile height does not
    apply, but the ranges do).  ``_pair_parts_tuned`` says what is in use: (ranges, ranges, row tiles per wave).
    Then, at 8, 32, 64 and 128 rows (one count per class of rows), the launch with stationary activations is timed
    against the winner with one to six ranges of the shorter K (and as many times more of the longer), each
    with what reads its partial sums behind it (the norm that adds them, where the two products have one width; else
    a charge for the ranges' bytes): the fastest is fixed for the class, or the staged kernel where that is not
    beaten by 2 % (``_pair_stationary_tuned``)."""
    key = (tuple(w1.shape), tuple(w2.shape))
    if not PAIR_TUNE or key in _active.pair_parts or not may_time():
        return
    lib = ops.load_library()
    (N1, K1), (N2, K2) = w1.shape, w2.shape
    a0, b0 = ops.gemm_splitk_pair_parts(N1, K1, N2, K2)
    fix = lambda c: lib.pta_gemm_splitk_pair_fix(int(N1), int(K1), int(N2), int(K2), int(c[0]), int(c[1]), int(c[2]))
    forget = lambda: lib.pta_gemm_splitk_pair_fix(int(N1), int(K1), int(N2), int(K2), 0, 0, 1)
    fix_st = lambda cls, c: lib.pta_gemm_splitk_pair_fix_stationary(int(N1), int(K1), int(N2), int(K2), int(cls), int(c[0]), int(c[1]))
    for cls in range(len(ops.STATIONARY_CLASS_ROWS)):
        fix_st(cls, (0, 0))  # the launches timed first are the staged kernel's
    cands = [(a0, b0, 1)] + [(a, b, 1) for a in range(max(1, a0 - 1), a0 + 3) for b in range(max(1, b0 - 2), b0 + 3)
                             if (a, b) != (a0, b0)]
    tall = lambda p: sorted({max(1, p - 1), p, p + 1, max(1, 2 * p - 1), 2 * p, 2 * p + 1})
    cands += [(a, b, 2) for a in tall(a0) for b in tall(b0)]
    cands = [c for c in cands if fix(c) == 0]
    xs = {rows: [torch.randn((rows, K), dtype=torch.float32, device=w1.device).to(torch.bfloat16) for K in (K1, K2)]
          for rows in sorted({PAIR_TUNE_ROWS, 24, 8, 32, 64, 128})}
    xs_bf16 = {rows: torch.zeros((rows, N1), dtype=torch.bfloat16, device=w1.device) for rows in xs}
    kmin = min(K1, K2)
    f1, f2 = max(1, (K1 + kmin // 2) // kmin), max(1, (K2 + kmin // 2) // kmin)
    st_cands = [(b * f1, b * f2) for b in (1, 2, 3, 4, 6) if b * f1 <= 16 and b * f2 <= 16 and fix_st(0, (b * f1, b * f2)) == 0]
    fix_st(0, (0, 0))
    most = [max([c[i] for c in cands] + [c[i] for c in st_cands] + [16]) for i in (0, 1)]
    parts = [torch.empty((most[i], 128, N), dtype=torch.float32, device=w1.device) for i, N in enumerate((N1, N2))]
    # A launch is timed over several copies of the matrices in turn (more bytes than the memory-side cache holds),
    # back to back between two events: every launch reads its matrices from memory, as in a model, and no gap of
    # the host's lies inside the timed span.
    copy_bytes = (w1.numel() + w2.numel()) * 2
    n_copies = max(2, min(6, int(640e6 // copy_bytes) + 1))
    copies = [(w1, w2)] + [(w1.clone(), w2.clone()) for _ in range(n_copies - 1)]

    def timed_ways(chosen, rows, rounds=3, fix=fix, read=None):
        best = [float("inf")] * len(chosen)
        for r in range(rounds + 1):  # the first round warms up
            for j, c in enumerate(chosen):
                fix(c)
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for a, b in copies:
                    ops._call("pta_gemm_splitk_pair_bf16", ops._ptr(parts[0]), ops._ptr(xs[rows][0]), ops._ptr(a), int(N1), int(K1),
                          ops._ptr(parts[1]), ops._ptr(xs[rows][1]), ops._ptr(b), int(N2), int(K2), rows, ops._stream())
                    if read is not None:
                        read(c, rows)
                end.record()
                end.synchronize()
                if r > 0:
                    best[j] = min(best[j], start.elapsed_time(end) / len(copies))
        return best

    # Two products of the same width are a block's last ones, and what reads their partial sums next is the norm
    # that adds them: it is launched behind every timed launch of the comparison below, so that a launch pays for
    # the ranges it leaves to be added and for how it leaves them (all at once at its end, or as it goes).
    norm_w = (torch.ones(N1, dtype=torch.float32, device=w1.device)
              if N1 == N2 and ops.layernorm_sum_ok(N1) and os.environ.get("PTA_PAIR_TUNE_READER", "1") != "0" else None)

    def read_sums(c, rows):
        views = [parts[i].view(-1)[:int(c[-2 + i]) * rows * N].view(int(c[-2 + i]), rows, N) for i, N in enumerate((N1, N2))]
        ops.layernorm_sum([(views[1], None), (views[0], None), xs_bf16[rows]], N1, w=norm_w, b=norm_w, eps=1e-5)

    try:
        times = timed_ways(cands, PAIR_TUNE_ROWS)
        order = sorted(range(len(cands)), key=lambda i: times[i])
        short = [0] + [i for i in order if i != 0 and times[i] < PAIR_TUNE_MARGIN * times[0]][:3]
        small = timed_ways([cands[i] for i in short], 24) if len(short) > 1 else [0.0]
    finally:
        forget()
    if os.environ.get("PTA_TUNE_VERBOSE"):
        print(f"[pta tune] pair {key}: rule {cands[0]} {times[0] * 1e3:.1f} us at {PAIR_TUNE_ROWS} rows; fastest " +
              ", ".join(f"{cands[i]} {times[i] * 1e3:.1f}" for i in order[:6]) +
              (f"; at 24 rows {[round(t * 1e3, 1) for t in small]} for {[cands[i] for i in short]}" if len(short) > 1 else ""),
              flush=True)
    chosen = cands[0]
    for i, t24 in zip(short[1:], small[1:]):  # fastest first
        if t24 <= 1.03 * small[0]:
            chosen = cands[i]
            break
    if chosen != cands[0]:
        fix(chosen)
    _active.pair_parts[key] = chosen
    # the launch with stationary activations against that choice, per class of rows
    chosen_st = []
    try:
        for cls, rows in enumerate((8, 32, 64, 128)):
            fix_st(cls, (0, 0))
            # what reads the partial sums afterwards pays for every range (measured: some 8 TB/s worth of them), so
            # a launch is charged for its ranges' bytes at that rate on top of its own time
            read = read_sums if norm_w is not None else None
            slices_ms = (lambda c: 0.0) if read else (lambda c: (c[0] * N1 + c[1] * N2) * rows * 4 / 8e12 * 1e3)
            t_staged = timed_ways([chosen[:2]], rows, fix=lambda c: None, read=read)[0] + slices_ms(chosen)
            t_st = (timed_ways([(cls,) + c for c in st_cands], rows, fix=lambda a: fix_st(a[0], a[1:]), read=read)
                    if st_cands else [])
            t_st = [t + slices_ms(c) for t, c in zip(t_st, st_cands)]
            # the fewest ranges among those within 1.5 % of the fastest: what separates them is less than a box
            # varies, and fewer ranges leave whatever reads them next less to read
            best = (min((i for i in range(len(st_cands)) if t_st[i] <= 1.015 * min(t_st)), key=lambda i: st_cands[i])
                    if st_cands else -1)
            keep = st_cands[best] if best >= 0 and t_st[best] < 0.98 * t_staged else (0, 0)
            chosen_st.append(keep)
            if os.environ.get("PTA_TUNE_VERBOSE"):
                print(f"[pta tune] pair {key} at {rows} rows (with the reading of the partial sums): staged {t_staged * 1e3:.1f} us; stationary " +
                      ", ".join(f"{c} {t * 1e3:.1f}" for c, t in zip(st_cands, t_st)) + f" -> {keep}", flush=True)
    finally:
        while len(chosen_st) < len(ops.STATIONARY_CLASS_ROWS):
            chosen_st.append((0, 0))
        for cls, c in enumerate(chosen_st):
            fix_st(cls, c)
    _active.pair_stationary[key] = tuple(chosen_st)


def gemm_splitk_pair_parts_rule(N1: int, K1: int, N2: int, K2: int):
    """The ranges of K that the kernel library's own rule gives a pair, whatever has been fixed for the shape."""
    lib = ops.load_library()
    kept = _active.pair_parts.get(((int(N1), int(K1)), (int(N2), int(K2))))
    lib.pta_gemm_splitk_pair_fix(int(N1), int(K1), int(N2), int(K2), 0, 0, 1)
    rule = ops.gemm_splitk_pair_parts(N1, K1, N2, K2)
    if kept is not None and tuple(kept) != rule + (1,):
        lib.pta_gemm_splitk_pair_fix(int(N1), int(K1), int(N2), int(K2), int(kept[0]), int(kept[1]), int(kept[2]))
    return rule


# Elements of both matrices of a pair launch up to which it beats the two products on their own beyond 48 rows.
# Measured in whole decode steps: pairs of 104 M elements (K = 4,544, N = 4,672 + 18,176) and of 92 M (K = 4,096, N
# = 6,144 + 16,384) win at every row count; a pair of 344 M (K = 8,192, N = 9,216 + 32,768) wins up to 48 rows (32
# rows: 20.8 against 23.0 ms a step) and loses beyond them to the vendor library's product for the longer matrix
# (64 rows: 24.3 against 23.3 ms).
PAIR_MAX_WEIGHTS = 160 * 1024 * 1024
PAIR_SURE_ROWS = 48


def pair_launch_pays(rows: int, w1: torch.Tensor, w2: torch.Tensor) -> bool:
    """Whether two products of ``rows`` rows (17 and more) run as one launch of the decode batch kernels."""
    return rows <= PAIR_SURE_ROWS or w1.numel() + w2.numel() <= PAIR_MAX_WEIGHTS
