"""Loads the gfx950 kernel library and declares its C entry points.

The library is loaded once per process. If it has not been built yet it is
built at the first call (hipcc must be present); there is no fallback: without
the library every op raises.
"""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_int, c_int64, c_float, c_void_p

from ..csrc import build as _build

_lock = threading.Lock()
_lib = None

P = c_void_p
I = c_int
F = c_float

_SIGNATURES = {
    "imparo_embed_gather": [P, I, P, P, I, I, I, P],
    "imparo_place_tokens": [P, P, P, P, I, I, P],
    "imparo_rms_norm": [P, P, I, I, P, P, P, I, I, I, F, I, P],
    "imparo_gemm": [P, P, P, P, I, I, I, I, I, I, I, P],
    "imparo_gemm_slices": [I, I, I, I],
    "imparo_gemm_adds": [I, I, I, I],
    "imparo_gemm_variant": [P, P, P, P, I, I, I, I, I, I, I, I, P],
    "imparo_short_conv_decode": [P, P, P, P, P, P, I, I, I, I, I, P],
    "imparo_in_proj_conv_decode": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, P],
    "imparo_qk_norm_rope_store": [P, P, P, F, P, I, I, P, P, P, I, I, P, P, P, I, I, I, I, I, I, I, I, P],
    "imparo_attention": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, I, I, P],
    "imparo_attention_decode": [P, P, P, P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P],
    # qkv, q_w, k_w, eps, inv_freq, n_freq, interleaved, k_cache, v_cache, write_kv, out, part_o, part_ml, rows, n_rows,
    # seg_start, positions, table, stride, page, heads, kv_heads, head_dim, n_pages, scale, window, n_splits, stream
    "imparo_attention_decode_qkv": [P, P, P, F, P, I, I, P, P, I, P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P],
    "imparo_attention_decode_qkv_takes": [I, I],
    "imparo_attention_decode_qkv_pays": [I, I],
    "imparo_attention_prefill": [P, P, P, P, P, P, I, P, I, I, P, P, P, P, I, I, I, I, I, I, F, I, P],
    "imparo_attention_prefill_splits": [I, I, I, I, I],
    "imparo_attention_decode_split": [],
    "imparo_attention_prefill_tile": [],
    "imparo_short_conv": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, P],
    "imparo_short_conv_state": [P, P, P, P, P, I, I, I, I, I, P],
    "imparo_argmax_rows": [P, P, I, I, P],
    "imparo_sample_rows": [P, P, P, P, I, I, P],
    "imparo_fill_f32": [P, F, c_int64, P],
    "imparo_fill_sites": [P, P, P, I, I, P],
    "imparo_attention_decode_static": [P, P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P],
    "imparo_load_code": [],
    "imparo_rows_parts": [I],
    # x, ssq_in, n_parts, eps, w, bias, y, out_dtype, x_io, ssq_out, weighted_out, weighted_by, m, n, k, epilogue, stream
    "imparo_rows_gemm": [P, P, I, F, P, P, P, I, P, P, P, P, I, I, I, I, P],
    "imparo_in_proj_conv_decode_normed": [P, P, I, F, P, P, P, P, P, P, P, I, I, I, I, I, I, P],
    "imparo_rows_fold_pays": [I, I, I],
    # a model's step as one call (kernels/program.py holds the structures)
    "imparo_program_new": ([I, I], P),
    "imparo_program_delete": ([P], None),
    "imparo_program_set_fold": [P, I],
    "imparo_program_embedding": [P, P, I, I, I],
    "imparo_program_norm": [P, P, F, I, I],
    "imparo_program_attention": [P, P],
    "imparo_program_short_conv": [P, P],
    "imparo_program_swiglu": [P, P],
    "imparo_program_head": [P, P, F, I, P],
    "imparo_program_n_regions": [P],
    "imparo_program_region_name": ([P, I], ctypes.c_char_p),
    "imparo_program_bind": [P, I, P, c_int64],
    "imparo_program_needs": [P, P, P],
    "imparo_program_run": [P, P, P, P],
    "imparo_program_error": ([P], ctypes.c_char_p),
}


class KernelLibraryError(RuntimeError):
    pass


def library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = _build.library_path()
        if not os.path.isfile(path):
            path = _rebuild("is not built")
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from e
        built_from = _hash_in(lib, "imparo_hip_source_hash")
        if built_from != _build.source_hash():
            # older than its sources (or from before libraries carried a hash): never used silently
            import _ctypes
            _ctypes.dlclose(lib._handle)
            path = _rebuild(f"at {path} was built from other sources ({built_from}) than those beside it")
            lib = ctypes.CDLL(path)
            if _hash_in(lib, "imparo_hip_source_hash") != _build.source_hash():
                raise KernelLibraryError(f"{path} still does not match its sources after a rebuild")
        for name, argtypes in _SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                raise KernelLibraryError(f"{path} lacks the entry point {name}; rebuild it "
                                         f"(python -m imparo_amd.csrc.build)") from None
            if isinstance(argtypes, tuple):          # (arguments, what it returns) where that is no status
                fn.argtypes, fn.restype = argtypes
            else:
                fn.argtypes, fn.restype = argtypes, c_int
        _lib = lib
        return _lib


def _hash_in(lib: ctypes.CDLL, name: str) -> str:
    try:
        fn = getattr(lib, name)
    except AttributeError:
        return "none"
    fn.restype = ctypes.c_char_p
    fn.argtypes = []
    return fn().decode("ascii", "replace")


def _rebuild(why: str) -> str:
    try:
        return _build.build(verbose=True)
    except Exception as e:  # no silent fallback: say why there is no library
        raise KernelLibraryError(f"the gfx950 kernel library {why} and building it failed: {e}") from e


def loaded_path() -> str:
    library()
    return _build.library_path()
