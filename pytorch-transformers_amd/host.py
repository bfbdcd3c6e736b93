"""Python face of the host runtime (``csrc/host/runtime_host.cpp``): loading and typed entry points.

The runtime is plain C++ with no GPU call; it holds the cache's bookkeeping (slots, page lists,
lengths) and lays a step's integer arrays out.  It is compiled at first use if no current build lies
beside the sources.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
ABI_VERSION = 4
OK, ERR_STEP, ERR_CACHE, ERR_FULL = 0, 1, 2, 3

_lib = None
_lock = threading.Lock()
_P_INT = ctypes.POINTER(ctypes.c_int)
_P_LL = ctypes.POINTER(ctypes.c_longlong)


def _build_module():
    spec = importlib.util.spec_from_file_location("_pta_csrc_build", os.path.join(_HERE, "csrc", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load():
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        b = _build_module()
        path = b.find_host_library(require_current=True) or b.build_host(verbose=True)
        lib = ctypes.CDLL(path)
        if lib.ptah_abi_version() != ABI_VERSION:
            raise RuntimeError(f"{path} has ABI {lib.ptah_abi_version()}, this package needs {ABI_VERSION}; rebuild it")
        lib.ptah_last_error.restype = ctypes.c_char_p
        lib.ptah_cache_new.restype = ctypes.c_void_p
        lib.ptah_cache_new.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _P_INT, _P_INT]
        lib.ptah_cache_delete.argtypes = [ctypes.c_void_p]
        lib.ptah_cache_delete.restype = None
        for name in ("ptah_alloc", "ptah_free_slots", "ptah_check"):
            getattr(lib, name).argtypes = [ctypes.c_void_p]
        for name in ("ptah_free", "ptah_is_live", "ptah_length", "ptah_free_pages", "ptah_held_pages"):
            getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_int]
        for name in ("ptah_reserve", "ptah_commit"):
            getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_int, _P_INT, _P_INT]
        lib.ptah_page_count.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        lib.ptah_pages.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, _P_INT]
        lib.ptah_plan_step.argtypes = [ctypes.c_void_p, ctypes.c_int, _P_INT, _P_INT, _P_LL, ctypes.c_int, ctypes.c_int,
                                       _P_INT, _P_INT, _P_INT]
        lib.ptah_decode_prepare.argtypes = [ctypes.c_void_p, ctypes.c_int, _P_INT, _P_LL, ctypes.c_int, _P_INT, _P_LL]
        lib.ptah_decode_fill.argtypes = [ctypes.c_void_p, ctypes.c_int, _P_INT, _P_LL, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        lib.ptah_commit_ones.argtypes = [ctypes.c_void_p, ctypes.c_int, _P_INT]
        lib.ptah_plan_data.argtypes = [ctypes.c_void_p]
        lib.ptah_plan_data.restype = _P_INT
        _lib = lib
        return lib


def last_error() -> str:
    return load().ptah_last_error().decode("utf-8", "replace")


def int_array(values):
    """A C int array from a sequence of Python ints."""
    return (ctypes.c_int * len(values))(*values)
