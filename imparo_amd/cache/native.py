"""Loads the host runtime library (page pools, cache manager, step packing)
and declares its C entry points. Built with the C++ compiler at first use if
it is not there; no GPU is needed for it."""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import POINTER, c_float, c_int, c_int32, c_int64, c_uint64, c_void_p

from ..csrc import build as _build

_lock = threading.Lock()
_lib = None

I, P = c_int, c_void_p
PI32, PI64 = POINTER(c_int32), POINTER(c_int64)

_SIGNATURES = {
    "imparo_pool_new": ([I], P), "imparo_pool_delete": ([P], None), "imparo_pool_alloc": ([P], I),
    "imparo_pool_free": ([P, I], I), "imparo_pool_n_free": ([P], I), "imparo_pool_n_pages": ([P], I),
    "imparo_pool_high_water": ([P], I), "imparo_pool_is_free": ([P, I], I), "imparo_pool_scramble": ([P, c_uint64], I),
    "imparo_cache_new": ([I, P, I, P, I], P), "imparo_cache_delete": ([P], None),
    "imparo_cache_group_pool": ([P, I], P), "imparo_cache_slot_pool": ([P], P),
    "imparo_cache_admit": ([P, c_int64], I), "imparo_cache_release": ([P, c_int64], I),
    "imparo_cache_reserve": ([P, c_int64, I], I), "imparo_cache_rollback": ([P, c_int64], I),
    "imparo_cache_commit": ([P, c_int64, I], I), "imparo_cache_is_live": ([P, c_int64], I),
    "imparo_cache_length": ([P, c_int64], I), "imparo_cache_slot": ([P, c_int64], I),
    "imparo_cache_table_len": ([P, I, c_int64], I), "imparo_cache_table_copy": ([P, I, c_int64, P, I], I),
    "imparo_cache_pages_needed": ([P, c_int64, I, P], I), "imparo_cache_first_needed_page": ([P, I, I], I),
    "imparo_cache_n_live": ([P], I), "imparo_cache_live_requests": ([P, P, I], I), "imparo_cache_check": ([P], I),
    "imparo_cache_pack": ([P, I, P, P, P, P, P, I, P, c_int64, P], c_int64),
    "imparo_cache_begin_step": ([P, I, P, P, P, P, P, I, I, P, P], I),
    "imparo_cache_abort_step": ([P, I, P, P], I), "imparo_cache_end_step": ([P, I, P, P], I),
    "imparo_sched_new": ([P, I, I, I], P), "imparo_sched_delete": ([P], None),
    "imparo_sched_add": ([P, c_int64, I, I], I),
    "imparo_sched_plan": ([P, P, P, P, P, I, P, P, I, P], I),
    "imparo_sched_advance": ([P], None), "imparo_sched_token": ([P, c_int64, I], I),
    "imparo_sched_drop_waiting_head": ([P, P], I), "imparo_sched_retract": ([P, c_int64], I),
    "imparo_sched_n_waiting": ([P], I), "imparo_sched_n_running": ([P], I),
    "imparo_sched_waiting": ([P, P, I], I), "imparo_sched_running": ([P, P, I], I),
    # plain float32 statements of the kernels, for tests (imparo_amd/kernels/reference.py)
    "imparo_ref_embed": ([P, P, P, I, I], None), "imparo_ref_rms_norm": ([P, P, c_float, P, I, I], None),
    "imparo_ref_gemm": ([P, P, P, P, I, I, I], None), "imparo_ref_swiglu": ([P, P, P, c_int64], None),
    "imparo_ref_head_norm_rope": ([P, P, c_float, P, P, I, P, I, I, I], None),
    "imparo_ref_attention": ([P, P, P, P, P, I, I, I, I, c_float, I], None),
    "imparo_ref_short_conv": ([P, P, P, P, P, I, I, I], None),
    "imparo_ref_argmax": ([P, P, I, I], None), "imparo_ref_sample": ([P, P, P, P, I, I], None),
}
EV_ADMIT, EV_WAIT, EV_PREEMPT, EV_FAIL = 1, 2, 3, 4

E_OUT_OF_PAGES, E_NOT_LIVE, E_ALREADY_LIVE, E_SHRINK, E_DOUBLE_FREE, E_RANGE, E_BUSY, E_CAPACITY = range(-1, -9, -1)
E_LOST_PAGE, E_SHARED_PAGE, E_SLOTS = -9, -10, -11
E_TWICE, E_EMPTY, E_POSITIONS, E_TOKEN, E_WANT = -12, -13, -14, -15, -16


def _built_from(lib: ctypes.CDLL) -> str:
    try:
        fn = lib.imparo_host_source_hash
    except AttributeError:
        return "none"
    fn.restype = ctypes.c_char_p
    fn.argtypes = []
    return fn().decode("ascii", "replace")


def host_library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = _build.host_library_path()
        if not os.path.isfile(path):
            path = _build.build_host(verbose=True)
        lib = ctypes.CDLL(path)
        if _built_from(lib) != _build.host_source_hash():
            # a library older than its sources: the host runtime needs no GPU and builds in seconds
            import _ctypes
            _ctypes.dlclose(lib._handle)
            path = _build.build_host(verbose=True)
            lib = ctypes.CDLL(path)
            if _built_from(lib) != _build.host_source_hash():
                raise RuntimeError(f"{path} still does not match its sources after a rebuild")
        for name, (argtypes, restype) in _SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                raise RuntimeError(f"{path} lacks the entry point {name}; rebuild it "
                                   f"(python -m imparo_amd.csrc.build)") from None
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
        return _lib
