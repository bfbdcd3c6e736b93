"""Python face of the HIP kernel library: loading, argument checks, one function per kernel.

There is no CPU fallback.  A function given a tensor that is not on a GPU, or
called when the library cannot be loaded, raises.  Shapes, strides and types are
checked here, before a pointer reaches a kernel.  Kernels run on torch's current
stream, so they order with torch's own work and are recorded by a HIP graph
capture like it.
"""
from __future__ import annotations

import ctypes
import functools
import importlib.util
import os
import threading
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
F32, BF16 = 0, 1
QKV_LAYOUT_CODES = {"grouped": 0, "tail": 1, "interleaved": 2}
# activations by the reference's names (src/transformers/activations.py:200-220) -> codes of csrc/common.h
ACT_CODES = {None: 0, "none": 0, "linear": 0, "gelu": 1, "gelu_python": 1, "gelu_new": 2, "gelu_pytorch_tanh": 2,
             "gelu_fast": 2, "gelu_accurate": 2, "quick_gelu": 3, "relu": 4, "relu2": 5, "relu6": 6, "silu": 7, "swish": 7,
             "sigmoid": 8, "tanh": 9, "leaky_relu": 10, "mish": 11, "gelu_10": 12, "laplace": 13}
ABI_VERSION = 9
PAIRING_CODES = {"half": 0, "interleaved": 1}  # PtaPairing: elements (i, i + rotary_dim / 2) or (2i, 2i + 1)
BIAS_OF_CODES = {"key": 0, "distance": 1}  # PtaBiasOf: the slope times the key's position, or times key - query position


class _PtaRotation(ctypes.Structure):
    _fields_ = [("inv_freq", ctypes.c_void_p), ("inv_freq_ld", ctypes.c_int), ("cs_scale", ctypes.c_float),
                ("rotary_dim", ctypes.c_int), ("pairing", ctypes.c_int)]


class _PtaScoreBias(ctypes.Structure):
    _fields_ = [("slopes", ctypes.c_void_p), ("of", ctypes.c_int), ("bf16", ctypes.c_int), ("scale", ctypes.c_float)]

_lib = None
_lock = threading.Lock()


class KernelError(RuntimeError):
    pass


from . import tuning  # noqa: E402  the timed choices; it calls the faces below back, so each refers to the other by module


def __getattr__(name: str):
    """Names of ``tuning`` (``decode_plan``, ``live_tuning``, ``tuning_table`` ...) are reachable here too."""
    if name.startswith("__"):
        raise AttributeError(name)
    try:
        return getattr(tuning, name)
    except AttributeError:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}") from None


def _build_module():
    spec = importlib.util.spec_from_file_location("_pta_csrc_build", os.path.join(_HERE, "csrc", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load_library(build_if_missing: bool = True):
    """Load libpta_kernels.so, compiling it first if no current build exists."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        b = _build_module()
        path = b.find_library(require_current=True)
        if path is None:
            if not build_if_missing:
                raise KernelError("libpta_kernels.so is not built (run __graft_entry__.build())")
            path = b.build(verbose=True)
        lib = ctypes.CDLL(path)
        lib.pta_last_error.restype = ctypes.c_char_p
        if lib.pta_abi_version() != ABI_VERSION:
            raise KernelError(f"{path} has ABI {lib.pta_abi_version()}, this package needs {ABI_VERSION}; rebuild it")
        _lib = lib
        return lib


def _call(name: str, *args) -> None:
    lib = load_library()
    if _timing is None or name in _HOST_ENTRIES:
        rc = getattr(lib, name)(*args)
    else:
        with timed(name, *_entry_cost(name, args)):
            rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.pta_last_error().decode("utf-8", "replace"))


# ---- per-kernel timings for measurements ----------------------------------------------------------------------
# With ``start_timing()`` every launch through this module (and the library products that ``timed`` wraps) is
# bracketed by two events; ``stop_timing()`` returns, per entry point, calls, microseconds, the bytes it has to
# read and the arithmetic it does.  Steps must then be launched directly (``model.use_graphs = False``): events
# cannot be recorded into a captured step.  ``timing_hint`` carries what an entry point's arguments do not say
# (how many cached keys and values an attention launch reads, the arithmetic of a prompt's attention).
_timing = None
_HOST_ENTRIES = ("pta_gemm_splitk_pair_parts", "pta_gemm_stationary_rule")  # entry points that launch nothing
timing_hint = {"attn_bytes": 0, "attn_flops": 0}


class timed:
    def __init__(self, name: str, nbytes: float = 0.0, flops: float = 0.0):
        self.name, self.nbytes, self.flops = name, nbytes, flops

    def __enter__(self):
        if _timing is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if _timing is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            _timing.append((self.name, self.start, end, self.nbytes, self.flops))
        return False


def start_timing() -> None:
    global _timing
    _timing = []


def stop_timing() -> dict:
    """``{entry point: {"calls", "us", "bytes", "flops"}}`` of everything launched since ``start_timing``."""
    global _timing
    records, _timing = _timing or [], None
    torch.cuda.synchronize()
    out: dict = {}
    for name, start, end, nbytes, flops in records:
        r = out.setdefault(name, {"calls": 0, "us": 0.0, "bytes": 0.0, "flops": 0.0})
        r["calls"] += 1
        r["us"] += start.elapsed_time(end) * 1e3
        r["bytes"] += nbytes
        r["flops"] += flops
    return out


def _entry_cost(name: str, a) -> tuple:
    """(bytes a launch has to read, arithmetic it does), from the entry point's own arguments: matrices count
    once, activations and results of a few rows are left out."""
    gemm = lambda M, N, K, elem=2: (float(N) * K * elem, 2.0 * M * N * K)
    both = lambda x, y: (x[0] + y[0], x[1] + y[1])
    if name == "pta_gemm_skinny_bf16":
        return gemm(a[6], a[7], a[8])
    if name == "pta_gemm_skinny_pair_bf16":
        return both(gemm(a[12], a[4], a[13]), gemm(a[12], a[10], a[13]))
    if name == "pta_gemm_skinny_pair_qkv_bf16":
        return both(gemm(a[22], (a[11] + 2 * a[12]) * a[13], a[23]), gemm(a[22], a[20], a[23]))
    if name == "pta_gemm_splitk_bf16":
        return gemm(a[7], a[8], a[9])
    if name == "pta_gemm_splitk_pair_bf16":
        return both(gemm(a[10], a[3], a[4]), gemm(a[10], a[8], a[9]))
    if name == "pta_gemm_splitk_pair_reduced_bf16":
        return both(gemm(a[16], a[5], a[6]), gemm(a[16], a[13], a[14]))
    if name == "pta_gemm_splitk_pair_reduced_qkv_bf16":
        return both(gemm(a[26], (a[13] + 2 * a[14]) * a[15], a[5]), gemm(a[26], a[23], a[24]))
    if name == "pta_gemm_splitk_reduced_qkv_bf16":
        return gemm(a[18], (a[13] + 2 * a[14]) * a[15], a[5])
    if name == "pta_gemm_f32":
        return gemm(a[6], a[7], a[8], 4)
    if name == "pta_layernorm_sum":
        return ((a[4] + a[7]) * float(a[17]) * a[19] * 4, 0.0)
    if name in ("pta_attn_mfma", "pta_attn_generic"):
        return (float(timing_hint.get("attn_bytes", 0)), float(timing_hint.get("attn_flops", 0)))
    return (0.0, 0.0)


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"dtype {dt} is not supported; use torch.float32 or torch.bfloat16")


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise KernelError(f"{name} is on {t.device}; the kernels run on the GPU only and there is no CPU fallback")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def _need_rows(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    """Like ``_need`` for a matrix whose rows may lie apart (a block of columns of a wider matrix)."""
    if isinstance(t, torch.Tensor) and t.dim() == 2 and t.is_cuda and not t.is_contiguous() and t.stride(1) == 1 \
            and t.stride(0) >= t.shape[1]:
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
        return
    _need(t, name, dtype, shape)


def _need_pools(k_pool, v_pool, dtype, nkv: int, d: int) -> None:
    """Key pages are [pages, kv_heads, 64, d]; value pages are transposed, [pages, kv_heads, d, 64]."""
    _need(k_pool, "k_pool", dtype)
    _need(v_pool, "v_pool", dtype)
    if tuple(k_pool.shape[1:]) != (nkv, 64, d) or k_pool.dim() != 4:
        raise KernelError(f"k_pool must be [pages, {nkv}, 64, {d}], got {tuple(k_pool.shape)}")
    if tuple(v_pool.shape) != (k_pool.shape[0], nkv, d, 64):
        raise KernelError(f"v_pool must be [{k_pool.shape[0]}, {nkv}, {d}, 64], got {tuple(v_pool.shape)}")


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[m] = table[ids[m]].  The caller has checked that ids lie in [0, rows)."""
    _need(table, "table")
    V, H = table.shape
    _need(ids, "ids", torch.int32)
    M = ids.numel()
    if out is None:
        out = torch.empty((M, H), dtype=table.dtype, device=table.device)
    _need(out, "out", table.dtype, (M, H))
    _call("pta_embed", _ptr(out), _ptr(table), _ptr(ids), M, H, dtype_code(table.dtype), _stream())
    return out


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, *, w2=None, b2=None,
              rows: Optional[torch.Tensor] = None):
    """LayerNorm of the rows of x (or of x[rows]); with (w2, b2) a second affine output of the same pass."""
    _need(x, "x")
    H = x.shape[-1]
    _need(w, "weight", torch.float32, (H,))
    _need(b, "bias", torch.float32, (H,))
    if rows is not None:
        _need(rows, "rows", torch.int32)
        M = rows.numel()
    else:
        M = x.shape[0]
    if x.dim() != 2:
        raise KernelError(f"x must be [tokens, features], got {tuple(x.shape)}")
    out1 = torch.empty((M, H), dtype=x.dtype, device=x.device)
    out2 = None
    if w2 is not None:
        _need(w2, "weight2", torch.float32, (H,))
        _need(b2, "bias2", torch.float32, (H,))
        out2 = torch.empty((M, H), dtype=x.dtype, device=x.device)
    if M == 0:
        return (out1, out2) if w2 is not None else out1
    _call("pta_layernorm", _ptr(out1), _ptr(out2), _ptr(x), _ptr(rows), _ptr(w), _ptr(b), _ptr(w2), _ptr(b2), M, H,
          ctypes.c_float(eps), dtype_code(x.dtype), _stream())
    return (out1, out2) if w2 is not None else out1


def epilogue_(y: torch.Tensor, bias=None, act=None, add1=None, add2=None) -> torch.Tensor:
    """In place: y = act(round(y + bias)) + add1 + add2.  The rows of y may lie apart."""
    _need_rows(y, "y")
    M, N = y.shape
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, a in (("add1", add1), ("add2", add2)):
        if a is not None:
            _need(a, name, y.dtype, (M, N))
    _call("pta_epilogue", _ptr(y), int(y.stride(0)), _ptr(bias), _ptr(add1), _ptr(add2), M, N, ACT_CODES[act],
          dtype_code(y.dtype), _stream())
    return y


def _rotation_arg(inv_freq, cs_scale: float, d: int, n_seqs: Optional[int] = None, rotary_dim: Optional[int] = None,
                  pairing: str = "half"):
    """The rotation of queries and keys as the kernels take it (a ``PtaRotation`` by reference; None: no rotation).
    ``inv_freq`` is one table ``[rotary_dim / 2]`` for all tokens or one per sequence of the step, ``[sequences,
    rotary_dim / 2]``; the first ``rotary_dim`` elements of a head (default: all of them) are rotated in pairs
    ``(i, i + rotary_dim / 2)`` (``"half"``) or ``(2i, 2i + 1)`` (``"interleaved"``)."""
    if inv_freq is None:
        return None
    r = int(d if rotary_dim is None else rotary_dim)
    problem = rotation_problem(d, rotary_dim, pairing)
    if problem is not None:
        raise KernelError(problem)
    _need(inv_freq, "inv_freq", torch.float32)
    if inv_freq.dim() == 1 and inv_freq.shape[0] == r // 2:
        ld = 0
    elif inv_freq.dim() == 2 and inv_freq.shape[1] == r // 2 and (n_seqs is None or inv_freq.shape[0] == n_seqs):
        ld = r // 2
    else:
        raise KernelError(f"inv_freq must be [{r // 2}] or [sequences, {r // 2}], got {tuple(inv_freq.shape)}")
    return ctypes.byref(_PtaRotation(inv_freq.data_ptr(), ld, float(cs_scale), r, PAIRING_CODES[pairing]))


def rotation_problem(d: int, rotary_dim: Optional[int] = None, pairing: str = "half") -> Optional[str]:
    """None if the launches that rotate take this arrangement, else why not (for refusing a model early)."""
    r = int(d if rotary_dim is None else rotary_dim)
    if pairing not in PAIRING_CODES:
        return f"a rotation with pairing {pairing!r} is not built; built: {sorted(PAIRING_CODES)}"
    if r < 2 or r % 2 or r > d:
        return f"rotary_dim must be even, from 2 up to the head size {d}; got {r}"
    return None


def score_bias_problem(bias_of: str, bf16: bool) -> Optional[str]:
    """None if the attention kernels form this bias on scores, else why not."""
    if bias_of not in BIAS_OF_CODES:
        return (f"a score bias of {bias_of!r} is not built; built: slopes per head times {sorted(BIAS_OF_CODES)} "
                "(the key's position, or its distance from the query)")
    if bf16 and bias_of != "key":
        return "rounding to bfloat16 as the reference rounds is built for slopes times the key's position only"
    return None


def _score_bias_arg(slopes, nh: int, bias_of: str = "key", bias_bf16: bool = True, bias_scale: float = 1.0):
    """A bias on attention scores as the kernels take it (a ``PtaScoreBias`` by reference; None: no bias):
    ``slopes[head] * x * bias_scale`` with x the key's position (``"key"``; ``bias_bf16``: position and product
    rounded to bfloat16 as the reference rounds them) or the key's position minus the query's (``"distance"``)."""
    if slopes is None:
        return None
    problem = score_bias_problem(bias_of, False)
    if problem is not None:
        raise KernelError(problem)
    _need(slopes, "slopes", torch.float32, (nh,))
    return ctypes.byref(_PtaScoreBias(slopes.data_ptr(), BIAS_OF_CODES[bias_of], int(bool(bias_bf16) and bias_of == "key"),
                                      float(bias_scale)))


def rope_dynamic_table(seq_start: torch.Tensor, cu_tokens: torch.Tensor, d: int, theta: float, factor: float,
                       max_pos: int) -> torch.Tensor:
    """A frequency table per sequence of the step, [sequences, d/2], for frequencies that follow the sequence's
    length after the step: the trained ones up to ``max_pos`` tokens, beyond that those of a base stretched by
    ``(factor * length / max_pos - (factor - 1)) ** (d / (d - 2))``."""
    n = seq_start.numel()
    _need(seq_start, "seq_start", torch.int32, (n,))
    _need(cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    out = torch.empty((n, d // 2), dtype=torch.float32, device=seq_start.device)
    _call("pta_rope_dynamic_table", _ptr(out), _ptr(seq_start), _ptr(cu_tokens), n, int(d), ctypes.c_float(theta),
          ctypes.c_float(factor), int(max_pos), _stream())
    return out


def qkv_rope_cache(fused: torch.Tensor, bias, inv_freq, cs_scale: float, token_pos, token_seq, block_table,
                   k_pool, v_pool, nh: int, nkv: int, d: int, layout: str, write_cache: bool = True,
                   rotary_dim: Optional[int] = None, pairing: str = "half") -> torch.Tensor:
    """Queries [M, nh, d] from the fused rows (which may lie apart); keys and values go to the cache pages.
    ``inv_freq``, ``rotary_dim`` and ``pairing`` say how queries and keys are rotated (``_rotation_arg``)."""
    M = fused.shape[0]
    _need_rows(fused, "fused", None, (M, (nh + 2 * nkv) * d))
    dt = fused.dtype
    if bias is not None:
        _need(bias, "bias", torch.float32, ((nh + 2 * nkv) * d,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, dt, nkv, d)
    q = torch.empty((M, nh, d), dtype=dt, device=fused.device)
    _call("pta_qkv_rope_cache", _ptr(q), _ptr(fused), int(fused.stride(0)), _ptr(bias), rot,
          _ptr(token_pos), _ptr(token_seq), _ptr(block_table), block_table.shape[1], _ptr(k_pool), _ptr(v_pool), M,
          nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache), dtype_code(dt), _stream())
    return q


def attention_sizes_problem(nh: int, nkv: int, d: int, rotated: bool) -> Optional[str]:
    """None if the attention kernels take these head counts and this head size (``rotated``: queries and keys are
    rotated by position), else the reason.  Launches nothing: for refusing a model before its weights are read."""
    lib = load_library()
    if lib.pta_attention_sizes_ok(int(nh), int(nkv), int(d), int(bool(rotated))) == 0:
        return None
    return lib.pta_last_error().decode("utf-8", "replace")


def attn_generic(q: torch.Tensor, k_pool, v_pool, block_table, token_seq, token_pos, slopes, scale: float,
                 window: int = 0, alibi_exact: bool = False, bias_of: str = "key", bias_scale: Optional[float] = None):
    """Causal attention of every token over its sequence's cache (the last ``window`` positions of it, itself
    included, if ``window`` > 0); out [M, nh*d].  ``slopes`` (None: no bias), ``bias_of``, ``alibi_exact`` (no
    rounding to bfloat16) and ``bias_scale`` (None: 1 / sqrt(head size), as the reference folds its bias into the
    mask) describe a bias on the scores (``_score_bias_arg``)."""
    _need(q, "q")
    M, nh, d = q.shape
    nkv = k_pool.shape[1]
    _need_pools(k_pool, v_pool, q.dtype, nkv, d)
    _need(block_table, "block_table", torch.int32)
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    bias = _score_bias_arg(slopes, nh, bias_of, not alibi_exact, d ** -0.5 if bias_scale is None else bias_scale)
    out = torch.empty((M, nh * d), dtype=q.dtype, device=q.device)
    _call("pta_attn_generic", _ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table),
          block_table.shape[1], _ptr(token_seq), _ptr(token_pos), bias, M, nh, nkv, d,
          ctypes.c_float(scale), int(window), dtype_code(q.dtype), _stream())
    return out


def gemm_f32(a: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None) -> torch.Tensor:
    """act(a @ w.T + bias) + add1 + add2 in true 32-bit with a fixed summation order."""
    _need(a, "a", torch.float32)
    _need(w, "w", torch.float32)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"a is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, t in (("add1", add1), ("add2", add2)):
        if t is not None:
            _need(t, name, torch.float32, (M, N))
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    _call("pta_gemm_f32", _ptr(out), _ptr(a), _ptr(w), _ptr(bias), _ptr(add1), _ptr(add2), M, N, K, ACT_CODES[act],
          _stream())
    return out


# The smallest range of keys that one wave of a split decode launch walks (PTA_ATTN_SPLIT and PTA_ATTN_TILES
# pin the cut of a decode launch for tuning: keys per wave, column tiles per wave).
ATTN_SPLIT_KEYS = 128
ATTN_FORCE_SPLIT = int(os.environ.get("PTA_ATTN_SPLIT", "0"))
ATTN_FORCE_TILES = int(os.environ.get("PTA_ATTN_TILES", "0"))
ATTN_FORCE_WIDE = int(os.environ.get("PTA_ATTN_WIDE", "-1"))  # eight-wave workgroups for prompts: 1 always, 0 never

def attn_mfma_ok(q: torch.Tensor) -> bool:
    """Whether the matrix-core attention kernel takes these queries (bfloat16, head size built)."""
    return q.dtype == torch.bfloat16 and bool(load_library().pta_attn_mfma_supported(int(q.shape[2])))


SHARED_KEYS = 0  # as the waves of a decode cut: the heads of a KV head share its keys in one workgroup


def attn_decode_shared_ok(head_dim: int, heads_per_kv_head: int) -> bool:
    """Whether a decode launch with keys shared through LDS is built for this shape (many heads on a KV head)."""
    return bool(load_library().pta_attn_decode_shared_ok(int(head_dim), int(heads_per_kv_head)))


def attn_mfma(q: torch.Tensor, k_pool, v_pool, block_table, cu_tokens, seq_start, slopes, scale: float, *,
              max_new: int, n_splits: int = 1, split_size: int = ATTN_SPLIT_KEYS, window: int = 0,
              decode_tiles: int = 0, decode_waves: int = 1, alibi_exact: bool = False,
              prompt_wide: Optional[bool] = None, bias_of: str = "key", bias_scale: Optional[float] = None) -> torch.Tensor:
    """Causal attention of a step's tokens over the cache on the matrix cores; out [M, nh*d].

    ``max_new`` bounds the new tokens of any sequence of the step; with ``n_splits > 1`` the keys
    are split into ranges of ``split_size`` and ``n_splits * split_size`` bounds every context.
    ``decode_tiles``: groups of sixteen heads of one KV head that a wave holds when ``max_new`` is 1
    (0: as many as the head size allows).  ``decode_waves``: waves of a workgroup that divide its keys among
    them, or ``SHARED_KEYS``: the heads of a KV head on the waves of one workgroup, which share its keys through
    LDS (``attn_decode_shared_ok``).  ``prompt_wide``: workgroups of eight waves (True) or four (False) for prompts
    with heads up to 64 (None: eight where the launch has workgroups enough).  ``slopes``, ``alibi_exact``,
    ``bias_of`` and ``bias_scale``: the bias on the scores, as in ``attn_generic``."""
    _need(q, "q", torch.bfloat16)
    M, nh, d = q.shape
    nkv = k_pool.shape[1]
    _need_pools(k_pool, v_pool, q.dtype, nkv, d)
    _need(block_table, "block_table", torch.int32)
    n_seqs = block_table.shape[0]
    _need(cu_tokens, "cu_tokens", torch.int32, (n_seqs + 1,))
    _need(seq_start, "seq_start", torch.int32, (n_seqs,))
    bias = _score_bias_arg(slopes, nh, bias_of, not alibi_exact, d ** -0.5 if bias_scale is None else bias_scale)
    out = torch.empty((M, nh * d), dtype=q.dtype, device=q.device)
    po = pm = pl = None
    if n_splits > 1:
        po = torch.empty((M, nh, n_splits, d), dtype=torch.float32, device=q.device)
        pm = torch.empty((M, nh, n_splits), dtype=torch.float32, device=q.device)
        pl = torch.empty((M, nh, n_splits), dtype=torch.float32, device=q.device)
    _call("pta_attn_mfma", _ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), block_table.shape[1],
          _ptr(cu_tokens), _ptr(seq_start), bias, n_seqs, int(max_new), M, nh, nkv, d,
          ctypes.c_float(scale),
          int(split_size), int(n_splits), _ptr(po), _ptr(pm), _ptr(pl), int(window), int(decode_tiles), int(decode_waves),
          ATTN_FORCE_WIDE if prompt_wide is None else int(bool(prompt_wide)), _stream())
    return out



def attention(q: torch.Tensor, k_pool, v_pool, block_table, ctx, slopes, scale: float, window: int = 0,
              alibi_exact: bool = False, bias_of: str = "key", bias_scale: Optional[float] = None) -> torch.Tensor:
    """Attention of a step's tokens over the cache: picks the kernel for the step's shape and type.

    bfloat16 with a head size the matrix-core kernel is built for: that kernel, with the context
    split over several waves when every sequence brings one token; anything else: the 32-bit
    kernel."""
    if attn_mfma_ok(q):
        n_splits, size, tiles, waves = 1, ATTN_SPLIT_KEYS, 0, 1
        if ctx.is_decode:
            shape = (ctx.n_seqs, q.shape[1], k_pool.shape[1], q.shape[2], ctx.max_len, getattr(ctx, "mean_len", 0))
            if window == 0:
                tuning.note_decode_launch(*shape)
            tiles, size, waves = tuning.decode_plan(*shape)
            n_splits = (ctx.max_len + size - 1) // size
        return attn_mfma(q, k_pool, v_pool, block_table, ctx.cu_tokens, ctx.seq_start, slopes, scale,
                         max_new=max(ctx.new_tokens), n_splits=n_splits, split_size=size, window=window,
                         decode_tiles=tiles, decode_waves=waves, alibi_exact=alibi_exact, bias_of=bias_of,
                         bias_scale=bias_scale)
    return attn_generic(q, k_pool, v_pool, block_table, ctx.token_seq, ctx.token_pos, slopes, scale, window, alibi_exact,
                        bias_of, bias_scale)


def sample(logits: torch.Tensor, *, do_sample: bool, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0,
           min_p: float = 0.0, typical_p: float = 1.0, epsilon_cutoff: float = 0.0, eta_cutoff: float = 0.0,
           penalty: float = 1.0, hist=None, hist_off=None, ban=None, ban_off=None, eos=None, suppress=None,
           remove_invalid: bool = False, renorm: bool = False, seed: int = 0, rng_seq=None, rng_step=None,
           uniforms=None, need_scores: bool = True, bias_tok=None, bias_val=None, bias_off=None, forced=None,
           decay: Optional[float] = None):
    """Processors and choice for every row of ``logits`` [R, V] (32-bit); returns (tokens int32 [R], scores [R, V]).

    ``bias_tok`` / ``bias_val`` / ``bias_off``: per row a list of tokens (each once) whose scores get a value added
    before every other processor.  ``forced``: token ids of which one is forced in this step (every other score
    goes, theirs become 0; a banned token stays gone).  ``decay``: the scores of the ``eos`` tokens gain
    ``|score| * decay`` after the removal of invalid values.

    Without ``need_scores``, a greedy choice that no processor touches is a plain argmax and the scores
    come back as None."""
    _need(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise KernelError(f"logits must be [rows, vocab], got {tuple(logits.shape)}")
    R, V = logits.shape
    if ban is not None and ban.numel() == 0:
        ban = ban_off = None  # no row has a banned token
    if bias_off is not None and (bias_tok is None or bias_tok.numel() == 0):
        bias_tok = bias_val = bias_off = None  # no row has a biased token
    if (not need_scores and not do_sample and penalty == 1.0 and suppress is None and ban_off is None
            and not remove_invalid and not renorm and bias_off is None and forced is None and decay is None):
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        _call("pta_argmax", _ptr(out), _ptr(logits), R, V, _stream())
        return out, None
    for name, t, n in (("hist_off", hist_off, R + 1), ("ban_off", ban_off, R + 1), ("suppress", suppress, R), ("rng_seq", rng_seq, R),
                       ("rng_step", rng_step, R)):
        if t is not None:
            _need(t, name, torch.int32, (n,))
    if hist is not None:
        _need(hist, "hist", torch.int32)
    if ban_off is not None:
        if ban is None:
            raise KernelError("ban_off without ban")
        _need(ban, "ban", torch.int32)
    if eos is not None:
        _need(eos, "eos", torch.int32)
    if uniforms is not None:
        _need(uniforms, "uniforms", torch.float32, (R,))
    if bias_off is not None:
        _need(bias_off, "bias_off", torch.int32, (R + 1,))
        _need(bias_tok, "bias_tok", torch.int32)
        _need(bias_val, "bias_val", torch.float32, tuple(bias_tok.shape))
    if forced is not None:
        _need(forced, "forced", torch.int32)
    if decay is not None and (eos is None or eos.numel() == 0):
        raise KernelError("a bonus on the EOS tokens needs their ids")
    work = torch.empty_like(logits)
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _call("pta_sample", _ptr(out), _ptr(work), _ptr(logits), R, V, int(bool(do_sample)), ctypes.c_float(temperature),
          int(top_k), ctypes.c_float(top_p), ctypes.c_float(min_p), ctypes.c_float(typical_p),
          ctypes.c_float(epsilon_cutoff), ctypes.c_float(eta_cutoff), ctypes.c_float(penalty), _ptr(hist), _ptr(hist_off),
          _ptr(ban), _ptr(ban_off),
          _ptr(eos), 0 if eos is None else int(eos.numel()), _ptr(suppress), int(bool(remove_invalid)),
          int(bool(renorm)), ctypes.c_uint64(int(seed) & (2 ** 64 - 1)), _ptr(rng_seq), _ptr(rng_step), _ptr(uniforms),
          int(bool(need_scores)), _ptr(bias_tok), _ptr(bias_val), _ptr(bias_off), _ptr(forced),
          0 if forced is None else int(forced.numel()), int(decay is not None), ctypes.c_float(decay or 0.0), _stream())
    return out, (work if need_scores else None)



def library_mm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w.T`` in bfloat16 through the vendor library, in the pieces along M that were measured fastest."""
    M, N = x.shape[0], w.shape[0]
    with timed("library_mm", float(w.numel()) * 2, 2.0 * M * N * w.shape[1]):
        if not tuning.MM_CHUNKS or M < 512:
            return torch.mm(x, w.t())
        if (N, w.shape[1], (M + 63) // 64) not in tuning.active().mm_plans and not tuning.may_time():
            return torch.mm(x, w.t())
        out = torch.empty((M, N), dtype=x.dtype, device=x.device)
        plan = tuning.mm_plan(x, w, out)
        at = 0
        for rows in plan:
            torch.mm(x[at:at + rows], w.t(), out=out[at:at + rows])
            at += rows
        return out



# ---- the vendor library's product with K cut into a batch ------------------------------------------------
# Where K is long against N (the feed-forward's second matrix) and the rows are a few hundred, the library's
# kernel choice has too few tiles of the result to fill the chip: with K = 18,176 and N = 4,544, 512 rows take 225
# us, and 112 us as a batch of two products over the halves of K (32-bit partial sums, added in order by the kernel
# that also applies bias, activation and additions, so no epilogue launch follows).  Timed once per shape when
# timing is on; without an entry the plain product runs.
MM_KSPLIT = os.environ.get("PTA_MM_KSPLIT", "1") != "0"
MM_KSPLIT_MAX_ROWS = 1536  # at 2,048 rows the batch gained nothing alone and lost 3 % in a model (K = 32,768, N = 8,192)


def _k_batch(x: torch.Tensor, w: torch.Tensor, S: int) -> torch.Tensor:
    M, K = x.shape
    xb = x.unflatten(1, (S, K // S)).transpose(0, 1)   # [S, M, K/S], rows as far apart as x's
    wb = w.unflatten(1, (S, K // S)).permute(1, 2, 0)  # [S, K/S, N]
    return torch.bmm(xb, wb, out_dtype=torch.float32)


def library_mm_ksplit(x: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None):
    """``act(x @ w.T + bias) + add1 + add2`` through the library's batched product over ranges of K, where that
    was timed faster than its plain product (once per shape, by 64 rows); else None."""
    M, (N, K) = x.shape[0], w.shape
    if (not MM_KSPLIT or K < 2 * N or not (tuning.SPLITK_MAX_ROWS < M <= MM_KSPLIT_MAX_ROWS) or K % 32 or x.stride(1) != 1
            or not w.is_contiguous()):
        return None
    key = (N, K, (M + 63) // 64)
    S = tuning.active().mm_ksplit.get(key)
    if S is None:
        if not tuning.may_time():
            return None
        ways = [(1, lambda: library_mm(x, w))] + [(s, (lambda s=s: _k_batch(x, w, s))) for s in (2, 4) if K % (s * 8) == 0]
        best = tuning.time_ways_cold([run for _, run in ways], x.device)
        pick = min(range(len(ways)), key=lambda i: best[i])
        S = ways[pick][0] if best[pick] < 0.9 * best[0] else 1
        tuning.active().mm_ksplit[key] = S
    if S == 1:
        return None
    with timed("library_mm", float(w.numel()) * 2, 2.0 * M * N * K):
        part = _k_batch(x, w, S)
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, a in (("add1", add1), ("add2", add2)):
        if a is not None:
            _need(a, name, torch.bfloat16, (M, N))
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _call("pta_gemm_reduce_parts", _ptr(y), _ptr(part), _ptr(bias), _ptr(add1), _ptr(add2), M, N, S, ACT_CODES[act], 0,
          _stream())
    return y


def gemm_skinny_pair_bf16(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor, bias1=None, act1=None,
                          bias2=None, act2=None):
    """(act1(x1 @ w1.T + bias1), act2(x2 @ w2.T + bias2)) in one launch: few rows, one K, bfloat16."""
    for name, t in (("x1", x1), ("w1", w1), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M, K = x1.shape
    if tuple(x2.shape) != (M, K) or w1.dim() != 2 or w2.dim() != 2 or w1.shape[1] != K or w2.shape[1] != K:
        raise KernelError(f"a pair shares M and K: x1 {tuple(x1.shape)}, x2 {tuple(x2.shape)}, w1 {tuple(w1.shape)}, "
                          f"w2 {tuple(w2.shape)}")
    N1, N2 = w1.shape[0], w2.shape[0]
    if bias1 is not None:
        _need(bias1, "bias1", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    y1 = torch.empty((M, N1), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_skinny_pair_bf16", _ptr(y1), _ptr(x1), _ptr(w1), _ptr(bias1), N1, ACT_CODES[act1], _ptr(y2), _ptr(x2),
          _ptr(w2), _ptr(bias2), N2, ACT_CODES[act2], M, K, _stream())
    return y1, y2


def gemm_skinny_pair_qkv_ok(x: torch.Tensor, w_qkv: torch.Tensor, w2: torch.Tensor, d: int) -> bool:
    """Whether the pair launch for few rows can take a fused query_key_value projection to its end (rotation,
    queries, cache pages): bfloat16, at most 16 rows, head sizes that are multiples of 32.  PTA_QKV_TAIL=0
    switches it off."""
    return (QKV_TAIL and gemm_skinny_ok(x, w_qkv) and gemm_skinny_ok(x, w2) and d % 32 == 0 and d <= 256
            and w_qkv.shape[1] == w2.shape[1])


QKV_TAIL = os.environ.get("PTA_QKV_TAIL", "1") != "0"


def gemm_skinny_pair_qkv(x1: torch.Tensor, w_qkv: torch.Tensor, bias_qkv, inv_freq, cs_scale: float, token_pos,
                         token_seq, block_table, k_pool, v_pool, nh: int, nkv: int, d: int, layout: str,
                         write_cache: bool, x2: torch.Tensor, w2: torch.Tensor, bias2=None, act2=None,
                         rotary_dim: Optional[int] = None, pairing: str = "half"):
    """One launch for a decode step's two input products, the first a fused query_key_value projection taken to
    its end: returns (queries [M, nh, d] rotated, act2(x2 @ w2.T + bias2)); keys and values are in the cache pages,
    as ``qkv_rope_cache`` would have left them."""
    for name, t in (("x1", x1), ("w_qkv", w_qkv), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M, K = x1.shape
    N1, N2 = (nh + 2 * nkv) * d, w2.shape[0]
    if tuple(x2.shape) != (M, K) or tuple(w_qkv.shape) != (N1, K) or w2.dim() != 2 or w2.shape[1] != K:
        raise KernelError(f"a pair shares M and K: x1 {tuple(x1.shape)}, x2 {tuple(x2.shape)}, w_qkv {tuple(w_qkv.shape)} "
                          f"(wanted [{N1}, {K}]), w2 {tuple(w2.shape)}")
    if bias_qkv is not None:
        _need(bias_qkv, "bias_qkv", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, torch.bfloat16, nkv, d)
    q = torch.empty((M, nh, d), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_skinny_pair_qkv_bf16", _ptr(q), _ptr(x1), _ptr(w_qkv), _ptr(bias_qkv), rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table), block_table.shape[1], _ptr(k_pool),
          _ptr(v_pool), nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache), _ptr(y2), _ptr(x2), _ptr(w2), _ptr(bias2),
          N2, ACT_CODES[act2], M, K, _stream())
    return q, y2


def gemm_splitk_bf16(x: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None,
                     out_f32: bool = False, rt: int = 0, parts: int = 0, stage_blocks: int = 0,
                     depth: int = 0) -> torch.Tensor:
    """act(x @ w.T + bias) + add1 + add2 for a batch of at most 128 rows of bfloat16: x shared through LDS,
    K split over workgroups where N gives too few of them."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    M, K = x.shape
    N = w.shape[0]
    if w.dim() != 2 or w.shape[1] != K:
        raise KernelError(f"x is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, t in (("add1", add1), ("add2", add2)):
        if t is not None:
            _need(t, name, torch.bfloat16, (M, N))
    parts = int(load_library().pta_gemm_splitk_parts(N, K, int(parts), int(rt)))
    part = torch.empty((parts, M, N), dtype=torch.float32, device=x.device) if parts > 1 else None
    out = torch.empty((M, N), dtype=torch.float32 if out_f32 else torch.bfloat16, device=x.device)
    _call("pta_gemm_splitk_bf16", _ptr(out), _ptr(part), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), _ptr(add2), M, N, K,
          ACT_CODES[act], int(out_f32), int(rt), int(parts), int(stage_blocks), int(depth), 1, _stream())
    return out


def gemm_splitk_partial(x: torch.Tensor, w: torch.Tensor, rt: int = 0, parts: int = 0, stage_blocks: int = 0) -> torch.Tensor:
    """x @ w.T left as 32-bit partial sums over ranges of K, [ranges, M, N]: for a kernel that adds them
    in order while it reads them (``layernorm_sum``)."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    M, K = x.shape
    N = w.shape[0]
    if w.dim() != 2 or w.shape[1] != K:
        raise KernelError(f"x is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    parts = int(load_library().pta_gemm_splitk_parts(N, K, int(parts), int(rt)))
    part = torch.empty((parts, M, N), dtype=torch.float32, device=x.device)
    _call("pta_gemm_splitk_bf16", None, _ptr(part), _ptr(x), _ptr(w), None, None, None, M, N, K, 0, 0, int(rt),
          int(parts), int(stage_blocks), 0, 0, _stream())
    return part


def gemm_splitk_pair_parts(N1: int, K1: int, N2: int, K2: int, M: int = 0):
    """How many ranges of K each product of a pair launch of ``M`` rows is cut into (0: by the kernel that walks
    K in stages, whatever the rows; steps of 17 to 128 rows may run with the activations stationary, which has
    ranges of its own)."""
    p1, p2 = ctypes.c_int(0), ctypes.c_int(0)
    _call("pta_gemm_splitk_pair_parts", int(N1), int(K1), int(N2), int(K2), int(M), ctypes.byref(p1), ctypes.byref(p2))
    return p1.value, p2.value


STATIONARY_CLASS_ROWS = (16, 32, 64, 128)  # a pair launch's rows count by the first of these that holds them


def gemm_stationary_rule(N1: int, K1: int, N2: int, K2: int, cls: int):
    """(ranges, ranges) of K of the pair launch with stationary activations for rows of class ``cls`` (the index
    into ``STATIONARY_CLASS_ROWS``), by the rule."""
    q1, q2 = ctypes.c_int(0), ctypes.c_int(0)
    _call("pta_gemm_stationary_rule", int(N1), int(K1), int(N2), int(K2), int(cls), ctypes.byref(q1), ctypes.byref(q2))
    return q1.value, q2.value



def gemm_splitk_pair_partial(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor):
    """(x1 @ w1.T, x2 @ w2.T), both left as 32-bit partial sums, in one launch; the products share M."""
    for name, t in (("x1", x1), ("w1", w1), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M = x1.shape[0]
    if x2.shape[0] != M or w1.dim() != 2 or w2.dim() != 2 or w1.shape[1] != x1.shape[1] or w2.shape[1] != x2.shape[1]:
        raise KernelError(f"a pair shares M: x1 {tuple(x1.shape)}, w1 {tuple(w1.shape)}, x2 {tuple(x2.shape)}, "
                          f"w2 {tuple(w2.shape)}")
    (N1, K1), (N2, K2) = w1.shape, w2.shape
    tuning.tune_pair_parts(w1, w2)
    p1, p2 = gemm_splitk_pair_parts(N1, K1, N2, K2, M)
    part1 = torch.empty((p1, M, N1), dtype=torch.float32, device=x1.device)
    part2 = torch.empty((p2, M, N2), dtype=torch.float32, device=x1.device)
    _call("pta_gemm_splitk_pair_bf16", _ptr(part1), _ptr(x1), _ptr(w1), N1, K1, _ptr(part2), _ptr(x2), _ptr(w2), N2, K2,
          M, _stream())
    return part1, part2


def gemm_splitk_pair_bf16(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor, bias1=None, act1=None,
                          bias2=None, act2=None):
    """(act1(x1 @ w1.T + bias1), act2(x2 @ w2.T + bias2)) for a batch of up to 128 rows: one matrix launch for
    both products and one launch that adds their partial sums."""
    for name, t in (("x1", x1), ("w1", w1), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M = x1.shape[0]
    if x2.shape[0] != M or w1.dim() != 2 or w2.dim() != 2 or w1.shape[1] != x1.shape[1] or w2.shape[1] != x2.shape[1]:
        raise KernelError(f"a pair shares M: x1 {tuple(x1.shape)}, w1 {tuple(w1.shape)}, x2 {tuple(x2.shape)}, "
                          f"w2 {tuple(w2.shape)}")
    lib = load_library()
    (N1, K1), (N2, K2) = w1.shape, w2.shape
    if bias1 is not None:
        _need(bias1, "bias1", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    tuning.tune_pair_parts(w1, w2)
    p1, p2 = gemm_splitk_pair_parts(N1, K1, N2, K2, M)
    part1 = torch.empty((p1, M, N1), dtype=torch.float32, device=x1.device)
    part2 = torch.empty((p2, M, N2), dtype=torch.float32, device=x1.device)
    y1 = torch.empty((M, N1), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_splitk_pair_reduced_bf16", _ptr(y1), _ptr(part1), _ptr(x1), _ptr(w1), _ptr(bias1), N1, K1,
          ACT_CODES[act1], _ptr(y2), _ptr(part2), _ptr(x2), _ptr(w2), _ptr(bias2), N2, K2, ACT_CODES[act2], M, _stream())
    return y1, y2


def gemm_splitk_pair_qkv(x1: torch.Tensor, w_qkv: torch.Tensor, bias_qkv, inv_freq, cs_scale: float, token_pos,
                         token_seq, block_table, k_pool, v_pool, nh: int, nkv: int, d: int, layout: str,
                         write_cache: bool, x2: torch.Tensor, w2: torch.Tensor, bias2=None, act2=None,
                         rotary_dim: Optional[int] = None, pairing: str = "half"):
    """The pair launch of a decode batch (17 to 256 rows) with its first product a fused query_key_value projection
    taken to its end by the launch that adds the partial sums: returns (queries [M, nh, d] rotated,
    act2(x2 @ w2.T + bias2)); keys and values are in the cache pages, as ``qkv_rope_cache`` leaves them."""
    for name, t in (("x1", x1), ("w_qkv", w_qkv), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M = x1.shape[0]
    N1, (N2, K2), K1 = (nh + 2 * nkv) * d, w2.shape, x1.shape[1]
    if x2.shape[0] != M or tuple(w_qkv.shape) != (N1, K1) or x2.shape[1] != K2:
        raise KernelError(f"a pair shares M: x1 {tuple(x1.shape)}, w_qkv {tuple(w_qkv.shape)} (wanted [{N1}, {K1}]), "
                          f"x2 {tuple(x2.shape)}, w2 {tuple(w2.shape)}")
    if d % 2:
        raise KernelError(f"head size {d} must be even")
    if bias_qkv is not None:
        _need(bias_qkv, "bias_qkv", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, torch.bfloat16, nkv, d)
    tuning.tune_pair_parts(w_qkv, w2)
    p1, p2 = gemm_splitk_pair_parts(N1, K1, N2, K2, M)
    part1 = torch.empty((p1, M, N1), dtype=torch.float32, device=x1.device)
    part2 = torch.empty((p2, M, N2), dtype=torch.float32, device=x1.device)
    q = torch.empty((M, nh, d), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_splitk_pair_reduced_qkv_bf16", _ptr(q), _ptr(part1), _ptr(x1), _ptr(w_qkv), _ptr(bias_qkv), K1,
          rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table),
          block_table.shape[1], _ptr(k_pool), _ptr(v_pool), nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache),
          _ptr(y2), _ptr(part2), _ptr(x2), _ptr(w2), _ptr(bias2), N2, K2, ACT_CODES[act2], M, _stream())
    return q, y2


def gemm_splitk_qkv(x: torch.Tensor, w_qkv: torch.Tensor, bias_qkv, inv_freq, cs_scale: float, token_pos, token_seq,
                    block_table, k_pool, v_pool, nh: int, nkv: int, d: int, layout: str, write_cache: bool,
                    rotary_dim: Optional[int] = None, pairing: str = "half"):
    """A fused query_key_value projection of a decode batch (17 to 256 rows) on its own, taken to its end by the
    launch that adds its partial sums: returns the queries [M, nh, d] rotated; keys and values are in the cache
    pages, as ``qkv_rope_cache`` leaves them."""
    _need(x, "x", torch.bfloat16)
    _need(w_qkv, "w_qkv", torch.bfloat16)
    M, K = x.shape
    N = (nh + 2 * nkv) * d
    if tuple(w_qkv.shape) != (N, K):
        raise KernelError(f"w_qkv {tuple(w_qkv.shape)}: wanted [{N}, {K}] for x {tuple(x.shape)}")
    if d % 2:
        raise KernelError(f"head size {d} must be even")
    if bias_qkv is not None:
        _need(bias_qkv, "bias_qkv", torch.float32, (N,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, torch.bfloat16, nkv, d)
    part = torch.empty((int(load_library().pta_gemm_splitk_parts(N, K, 0, 0)), M, N), dtype=torch.float32, device=x.device)
    q = torch.empty((M, nh, d), dtype=torch.bfloat16, device=x.device)
    _call("pta_gemm_splitk_reduced_qkv_bf16", _ptr(q), _ptr(part), _ptr(x), _ptr(w_qkv), _ptr(bias_qkv), K,
          rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table),
          block_table.shape[1], _ptr(k_pool), _ptr(v_pool), nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache), M,
          _stream())
    return q


def gemm_partial_pair_ok(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor) -> bool:
    """Whether two products onto the same features are best left as partial sums of one launch: up to 128
    rows each, and at least one of them worth leaving so on its own."""
    return (_bf16_rows_ok(x1, w1) and _bf16_rows_ok(x2, w2) and 0 < x1.shape[0] == x2.shape[0] <= tuning.SPLITK_MAX_ROWS
            and tuning.splitk_rows_ok(x1, w1, w2)
            and w1.shape[0] == w2.shape[0] and w1.shape[0] % 8 == 0
            and (gemm_partial_ok(x1, w1) or gemm_partial_ok(x2, w2)))


def gemm_partial_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether leaving x @ w.T as partial sums for the next norm pays: up to 128 rows, and either K long against
    N (any batch: the kernel for few rows has too few row tiles there) or a batch past 16 rows."""
    if not (_bf16_rows_ok(x, w) and 0 < x.shape[0] <= tuning.SPLITK_MAX_ROWS and w.shape[0] % 8 == 0 and tuning.splitk_rows_ok(x, w)):
        return False
    return w.shape[1] >= 2 * w.shape[0] or (x.shape[0] > 16 and w.shape[0] < 2 * w.shape[1])


def layernorm_sum_ok(H: int) -> bool:
    return bool(load_library().pta_layernorm_sum_ok(int(H)))


def layernorm_sum_rows_min() -> int:
    """Rows from which a sum of tensors alone is formed and normalised by a wave per row (the arrangement for prompts)."""
    return int(load_library().pta_layernorm_sum_rows_min())


def layernorm_sum(terms, H: int, *, w=None, b=None, eps: float = 0.0, w2=None, b2=None, rows=None,
                  want_x: bool = True):
    """The sum of ``terms`` rounded to bfloat16 and, with (w, b), its LayerNorm: ``(x, out1, out2)``.

    A term is a bfloat16 tensor [M, H] or a pair (partial sums [P, M, H] in 32-bit, bias or None) of a
    product left unreduced; at most two products and three tensors, products first.  A product is valued as its
    own epilogue would have stored it; the terms are added in 32-bit in the order given, and the sum is rounded."""
    prods = [t for t in terms if isinstance(t, tuple)]
    adds = [t for t in terms if not isinstance(t, tuple)]
    if len(prods) > 2 or len(adds) > 3 or not terms:
        raise KernelError(f"layernorm_sum takes one to five terms, at most two products and three tensors; got {len(terms)}")
    if any(isinstance(t, tuple) for t in terms[len(prods):]):
        raise KernelError("layernorm_sum: products must come before tensors in the list of terms")
    M_in = None
    for part, bias in prods:
        _need(part, "partial sums", torch.float32)
        if part.dim() != 3 or part.shape[2] != H:
            raise KernelError(f"partial sums must be [parts, rows, {H}], got {tuple(part.shape)}")
        if bias is not None:
            _need(bias, "bias", torch.float32, (H,))
        M_in = part.shape[1] if M_in is None else M_in
        if part.shape[1] != M_in:
            raise KernelError("terms differ in their number of rows")
    for a in adds:
        _need(a, "addend", torch.bfloat16)
        M_in = a.shape[0] if M_in is None else M_in
        if tuple(a.shape) != (M_in, H):
            raise KernelError(f"addend must be [{M_in}, {H}], got {tuple(a.shape)}")
    ref = prods[0][0] if prods else adds[0]
    if rows is not None:
        _need(rows, "rows", torch.int32)
        M = rows.numel()
    else:
        M = M_in
    dev = ref.device
    norm = w is not None
    if norm:
        _need(w, "weight", torch.float32, (H,))
        _need(b, "bias", torch.float32, (H,))
    if w2 is not None:
        _need(w2, "weight2", torch.float32, (H,))
        _need(b2, "bias2", torch.float32, (H,))
    out_x = torch.empty((M, H), dtype=torch.bfloat16, device=dev) if want_x else None
    out1 = torch.empty((M, H), dtype=torch.bfloat16, device=dev) if norm else None
    out2 = torch.empty((M, H), dtype=torch.bfloat16, device=dev) if norm and w2 is not None else None
    if M == 0:
        return out_x, out1, out2
    pb, bb = prods[0] if prods else (None, None)  # the kernel adds B first, then A
    pa, ba = prods[1] if len(prods) > 1 else (None, None)
    a1 = adds[0] if adds else None
    a2 = adds[1] if len(adds) > 1 else None
    a3 = adds[2] if len(adds) > 2 else None
    _call("pta_layernorm_sum", _ptr(out_x), _ptr(out1), _ptr(out2), _ptr(pa), 0 if pa is None else pa.shape[0], _ptr(ba),
          _ptr(pb), 0 if pb is None else pb.shape[0], _ptr(bb), _ptr(a1), _ptr(a2), _ptr(a3), _ptr(rows), _ptr(w), _ptr(b),
          _ptr(w2), _ptr(b2), M_in, M, H, ctypes.c_float(eps), _stream())
    return out_x, out1, out2


def _bf16_rows_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the kernel for few rows takes this product and is the faster choice for it: bfloat16 with K a
    multiple of 8 and at most 16 rows (measured on MI355X against the vendor library at K = 4,544 and K = 18,176)."""
    return _bf16_rows_ok(x, w) and 0 < x.shape[0] <= 16


def gemm_splitk_pair_ok(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor) -> bool:
    """Whether the two products run as a pair launch of the decode batch kernel (17 to 256 rows; beyond 128 only
    where the pair was timed faster than the library's two products)."""
    return (_bf16_rows_ok(x1, w1) and _bf16_rows_ok(x2, w2) and 16 < x1.shape[0] == x2.shape[0] <= tuning.SPLITK_MAX_ROWS
            and tuning.splitk_rows_ok(x1, w1, w2))


def gemm_splitk_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the kernel for a decode batch of 17 to 128 rows is the faster choice.  Measured at K = 4,544 and
    K = 18,176: it beats the vendor library except where N is long against K (the feed-forward's first matrix
    and the output head), which give the library enough row tiles to fill the chip."""
    return (_bf16_rows_ok(x, w) and 16 < x.shape[0] <= tuning.SPLITK_MAX_ROWS and w.shape[0] < 2 * w.shape[1]
            and tuning.splitk_rows_ok(x, w))


def gemm_skinny_bf16(x: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None,
                     out_f32: bool = False, variant: int = 0, waves: int = 0) -> torch.Tensor:
    """act(x @ w.T + bias) + add1 + add2 for at most 64 rows of bfloat16, 32-bit accumulation."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"x is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, t in (("add1", add1), ("add2", add2)):
        if t is not None:
            _need(t, name, torch.bfloat16, (M, N))
    out = torch.empty((M, N), dtype=torch.float32 if out_f32 else torch.bfloat16, device=x.device)
    _call("pta_gemm_skinny_bf16", _ptr(out), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), _ptr(add2), M, N, K,
          ACT_CODES[act], int(out_f32), int(variant), int(waves), _stream())
    return out
