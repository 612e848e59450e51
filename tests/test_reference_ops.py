"""The plain C++ statements of the kernels (imparo_amd/csrc/host/reference_ops.cpp) against the
plain Python implementation and against the vectors the reference's own tests hold. Two texts
written apart, from the same formulas: where they agree, a kernel checked against either is
checked against both. No GPU is needed."""
import math

import numpy as np
import pytest
import torch

import plain_lfm2 as P
from imparo_amd.kernels import reference as R


def rnd(*shape, seed=0, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale)


def close(a, b, tol=1e-5):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape
    assert np.abs(a - b).max() <= tol * max(1.0, np.abs(b).max()), np.abs(a - b).max()


def test_embedding_and_norm_and_products():
    table, ids = rnd(11, 6, seed=1), [3, 0, 10, 3]
    assert np.array_equal(R.embed(table, ids), table[ids].numpy())
    with pytest.raises(ValueError):
        R.embed(table, [11])
    x, w = rnd(5, 37, seed=2), 1 + 0.1 * rnd(37, seed=3)
    close(R.rms_norm(x, w, 1e-5), P.rms_norm(x, w, 1e-5))
    close(R.rms_norm(7.0 * x, w, 1e-6), P.rms_norm(x, w, 1e-6), 1e-4)          # scale-invariant up to eps
    wt, b = rnd(13, 37, seed=4), rnd(13, seed=5)
    close(R.gemm(x, wt, b), P.linear(x, wt, b))
    close(R.gemm(x, wt), x.double() @ wt.double().t())
    # the activation sits on the gate: silu(1) = 0.7310586, silu(0) = 0
    # (/root/reference/crates/imparo-cuda/native/tests/lfm2_ops_test.cpp:83-84)
    assert abs(float(R.swiglu([1.0], [1.0])[0]) - 0.7310586) < 1e-6 and float(R.swiglu([0.0], [5.0])[0]) == 0.0
    g, u = rnd(4, 9, seed=6), rnd(4, 9, seed=7)
    close(R.swiglu(g, u), P.silu(g) * u)
    assert not np.allclose(R.swiglu(g, u), R.swiglu(u, g))


def test_rotation_and_head_norm():
    T, H, D, base = 7, 3, 16, 50000.0
    x, w = rnd(T, H, D, seed=1), 1 + 0.1 * rnd(D, seed=2)
    positions = [0, 1, 5, 100, 4000, 4001, 77777]
    inv = np.power(np.float32(base), (np.float32(-2.0) * np.arange(D // 2, dtype=np.float32) / np.float32(D))).astype(np.float32)
    close(R.head_norm_rope(x, w, 1e-5, positions, inv), P.rope_neox(P.rms_norm(x, w, 1e-5), positions, base, D), 2e-5)
    # position 0 is the identity; no table, no rotation
    close(R.head_norm_rope(x[:1], None, 0.0, [0], inv), x[:1])
    close(R.head_norm_rope(x, w, 1e-5, positions, None), P.rms_norm(x, w, 1e-5))
    # a partial rotation leaves the other dims alone, and pairs are (i, i + n_freq)
    inv6 = np.power(np.float32(base), (np.float32(-2.0) * np.arange(3, dtype=np.float32) / np.float32(6))).astype(np.float32)
    part = R.head_norm_rope(x, None, 0.0, positions, inv6)
    close(part, P.rope_neox(x, positions, base, 6), 2e-5)
    assert np.array_equal(part[..., 6:], x.numpy()[..., 6:]) and not np.allclose(part[1:, :, :6], x.numpy()[1:, :, :6])
    one = torch.zeros(1, 1, 6)
    one[0, 0, 0] = 1.0
    got = R.head_norm_rope(one, None, 0.0, [1], np.array([math.pi / 2, 0.0, 0.0], dtype=np.float32))
    close(got[0, 0], [0.0, 0.0, 0.0, 1.0, 0.0, 0.0], 1e-6)        # x0 -> x0 cos - x3 sin, x3 -> x0 sin + x3 cos


def test_attention():
    # /root/reference/crates/imparo-model/src/cpu_support.rs:485-512:
    # q = [1,0] twice, k = [[0,1],[1,0]], v = I: row 0 sees only key 0 -> [1,0]; row 1's weights sum to 1
    q = np.array([[[1.0, 0.0]], [[1.0, 0.0]]], dtype=np.float32)
    k = np.array([[[0.0, 1.0]], [[1.0, 0.0]]], dtype=np.float32)
    v = np.array([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=np.float32)
    out = R.attention(q, k, v, [0, 1], 1.0)
    assert out[0, 0].tolist() == [1.0, 0.0] and abs(out[1, 0].sum() - 1.0) < 1e-6 and out[1, 0, 1] > out[1, 0, 0]
    T, H, Hk, D = 23, 6, 2, 8
    qq, kk, vv = rnd(T, H, D, seed=1), rnd(T, Hk, D, seed=2), rnd(T, Hk, D, seed=3)
    for window in (None, 5, 1):
        close(R.attention(qq, kk, vv, range(T), 0.3, window), P.attend(qq, kk, vv, range(T), 0.3, window))
    # the last queries alone, against keys that are already there
    close(R.attention(qq[-4:], kk, vv, range(T - 4, T), 0.3, 7), P.attend(qq, kk, vv, range(T), 0.3, 7)[-4:])
    # contiguous groups of heads share a kv head (not interleaved): head 2 reads kv head 0, head 3 kv head 1
    vv2 = vv.clone()
    vv2[:, 1] += 100.0
    delta = R.attention(qq, kk, vv2, range(T), 0.3) - R.attention(qq, kk, vv, range(T), 0.3)
    assert np.abs(delta[:, :3]).max() == 0.0 and np.abs(delta[:, 3:] - 100.0).max() < 1e-3
    with pytest.raises(ValueError):
        R.attention(qq, kk[:5], vv[:5], range(T), 0.3)


def test_short_conv():
    # tap 0 meets the oldest value (/root/reference/crates/imparo-cpu/src/ops.rs:1207-1254)
    bcx = np.ones((2, 3), dtype=np.float32)
    y, s = R.short_conv(bcx, [[1.0, 0.0, 0.0]], None, [[5.0], [7.0]])
    assert y.flatten().tolist() == [5.0, 7.0] and s.flatten().tolist() == [1.0, 1.0]
    y, _ = R.short_conv(bcx, [[0.0, 0.0, 1.0]], None, [[5.0], [7.0]])
    assert y.flatten().tolist() == [1.0, 1.0]
    # /root/reference/crates/imparo-cuda/native/tests/lfm2_ops_test.cpp:46-62
    y, s = R.short_conv([[2.0, 0.0, 3.0], [2.0, 0.0, 5.0]], [[1.0, 0.0, 0.0, 0.0]], None, [[11.0], [13.0], [17.0]])
    assert y.flatten().tolist() == [0.0, 0.0] and s.flatten().tolist() == [17.0, 6.0, 10.0]
    E, L, T = 10, 4, 9
    bcx, w, b = rnd(T, 3 * E, seed=1), rnd(E, L, seed=2), rnd(E, seed=3)
    state = rnd(L - 1, E, seed=4)
    y_ref, s_ref = P.short_conv(bcx, w.reshape(E, 1, L), b, state)
    y, s = R.short_conv(bcx, w, b, state)
    close(y, y_ref)
    close(s, s_ref)
    # a segment equals the same tokens one at a time, outputs and state exactly
    st, ys = state.numpy().copy(), []
    for t in range(T):
        yt, st = R.short_conv(bcx[t:t + 1], w, b, st)
        ys.append(yt)
    assert np.array_equal(np.concatenate(ys), y) and np.array_equal(st, s)


def test_picking_tokens():
    nan = float("nan")
    rows = [[1.0, 3.0, 3.0, 2.0], [nan, -1.0, nan, -1.0], [nan, nan, nan, nan], [-np.inf, -np.inf, 0.0, 0.0]]
    assert R.argmax(rows).tolist() == [1, 1, 0, 2]
    big = rnd(5, 1000, seed=1)
    assert R.argmax(big).tolist() == [P.argmax_first(r) for r in big]
    # inverse CDF over softmax(logits / T): uniform 0 picks the first token with weight, just under 1 the last
    logits = np.log(np.array([[0.1, 0.2, 0.3, 0.4]], dtype=np.float32))
    for u, want in ((0.0, 0), (0.05, 0), (0.15, 1), (0.299, 1), (0.31, 2), (0.59, 2), (0.61, 3), (0.9999, 3)):
        assert R.sample(logits, [1.0], [u]).tolist() == [want]
    assert R.sample(logits, [0.0], [0.7]).tolist() == [3]          # temperature 0 is the argmax
    sharp = R.sample(np.repeat(logits, 50, 0), [0.05] * 50, np.linspace(0.01, 0.99, 50))
    assert (sharp == 3).mean() > 0.9                               # a low temperature concentrates on the top
    row = rnd(1, 300, seed=2).numpy()
    cdf = np.cumsum(np.exp((row[0].astype(np.float64) - row.max()) / 0.8))
    for u in (0.03, 0.42, 0.77):
        assert R.sample(row, [0.8], [u]).tolist() == [int(np.searchsorted(cdf, u * cdf[-1], side="right"))]
