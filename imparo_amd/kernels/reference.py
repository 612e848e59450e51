"""NumPy faces of the plain C++ statements of the kernels
(csrc/host/reference_ops.cpp): float32, whole arrays, sums in the order k = 0, 1,
2, ... They run on the host, need no GPU, and exist for tests: every GPU kernel
is compared with the function here that states what it computes."""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np

from ..cache.native import host_library


def _f(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _i(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a: Optional[np.ndarray]) -> Optional[int]:
    return None if a is None else a.ctypes.data


def embed(table, ids) -> np.ndarray:
    table, ids = _f(table), _i(ids)
    if ids.size and (ids.min() < 0 or ids.max() >= table.shape[0]):
        raise ValueError("a token id is outside the table")
    out = np.empty((ids.shape[0], table.shape[1]), dtype=np.float32)
    host_library().imparo_ref_embed(_p(table), _p(ids), _p(out), ids.shape[0], table.shape[1])
    return out


def rms_norm(x, weight, eps: float) -> np.ndarray:
    x, weight = _f(x), _f(weight)
    out = np.empty_like(x)
    host_library().imparo_ref_rms_norm(_p(x), _p(weight), eps, _p(out), x.size // x.shape[-1], x.shape[-1])
    return out


def gemm(x, w, bias=None) -> np.ndarray:
    x, w = _f(x), _f(w)
    bias = None if bias is None else _f(bias)
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k:
        raise ValueError("inner sizes differ")
    out = np.empty((m, n), dtype=np.float32)
    host_library().imparo_ref_gemm(_p(x), _p(w), _p(bias), _p(out), m, n, k)
    return out


def swiglu(gate, up) -> np.ndarray:
    gate, up = _f(gate), _f(up)
    out = np.empty_like(gate)
    host_library().imparo_ref_swiglu(_p(gate), _p(up), _p(out), gate.size)
    return out


def head_norm_rope(x, weight, eps: float, positions, inv_freq) -> np.ndarray:
    """x [tokens, heads, head_dim]; weight [head_dim] or None; inv_freq [n_freq] or None."""
    x = _f(x)
    weight = None if weight is None else _f(weight)
    inv_freq = None if inv_freq is None else _f(inv_freq)
    positions = _i(positions)
    out = np.empty_like(x)
    host_library().imparo_ref_head_norm_rope(_p(x), _p(weight), eps, _p(positions), _p(inv_freq),
                                             0 if inv_freq is None else inv_freq.shape[0], _p(out), *x.shape)
    return out


def attention(q, k, v, q_positions, scale: float, window: Optional[int] = None) -> np.ndarray:
    """q [queries, heads, D]; k, v [keys, kv_heads, D] hold positions 0 .. keys-1 of one request."""
    q, k, v, q_positions = _f(q), _f(k), _f(v), _i(q_positions)
    if q_positions.size and q_positions.max() >= k.shape[0]:
        raise ValueError("a query's position has no key")
    out = np.empty_like(q)
    host_library().imparo_ref_attention(_p(q), _p(k), _p(v), _p(q_positions), _p(out), q.shape[0], q.shape[1],
                                        k.shape[1], q.shape[2], scale, int(window or 0))
    return out


def short_conv(bcx, weight, bias, state) -> Tuple[np.ndarray, np.ndarray]:
    """bcx [tokens, 3 width]; weight [width, taps]; state [taps-1, width]. Returns (y, new state)."""
    bcx, weight, state = _f(bcx), _f(weight), _f(state).copy()
    bias = None if bias is None else _f(bias)
    width, taps = weight.shape
    y = np.empty((bcx.shape[0], width), dtype=np.float32)
    host_library().imparo_ref_short_conv(_p(bcx), _p(weight), _p(bias), _p(state), _p(y), bcx.shape[0], width, taps)
    return y, state


def argmax(logits) -> np.ndarray:
    logits = _f(logits)
    out = np.empty(logits.shape[0], dtype=np.int32)
    host_library().imparo_ref_argmax(_p(logits), _p(out), *logits.shape)
    return out


def sample(logits, temperature, uniform) -> np.ndarray:
    logits, temperature, uniform = _f(logits), _f(temperature), _f(uniform)
    out = np.empty(logits.shape[0], dtype=np.int32)
    host_library().imparo_ref_sample(_p(logits), _p(temperature), _p(uniform), _p(out), *logits.shape)
    return out
