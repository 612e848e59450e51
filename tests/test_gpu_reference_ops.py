"""Each GPU kernel beside the plain C++ statement of what it computes
(imparo_amd/csrc/host/reference_ops.cpp through imparo_amd.kernels.reference).
Where the kernel sums in the statement's order (the float32 product, the short
convolution, the picks) the results are the same bits; where it sums in
parallel (norms, softmax) they agree to float32 rounding."""
import math

import numpy as np
import pytest
import torch

from gpu_helpers import hand_context
from imparo_amd.kernels import reference as R
from test_gpu_kernels import _attention_case, ops, rnd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("m,n,k", [(1, 40, 96), (7, 136, 264), (65, 200, 1032), (130, 70, 50)])
def test_float32_product_is_the_statement_bit_for_bit(m, n, k):
    x, w, b = rnd(m, k, seed=1), rnd(n, k, seed=2), rnd(n, seed=3)
    for bias in (None, b):
        out = torch.empty(m, n, device=DEV)
        ops().gemm(x.to(DEV), w.to(DEV), out, bias=None if bias is None else bias.to(DEV))
        assert np.array_equal(out.cpu().numpy(), R.gemm(x, w, bias))
    if k % 8:
        return                         # the bfloat16 kernels take inner sizes in steps of 8
    # bfloat16 operands accumulate in float32 in another order: float32 rounding of the sums apart
    xb, wb = x.to(torch.bfloat16), w.to(torch.bfloat16)
    out = torch.empty(m, n, device=DEV)
    ops().gemm(xb.to(DEV), wb.to(DEV), out)
    ref = R.gemm(xb.float(), wb.float())
    assert np.abs(out.cpu().numpy() - ref).max() <= 1e-6 * math.sqrt(k) * np.abs(ref).max()


def test_embedding_norm_and_gate():
    table = rnd(37, 24, seed=4)
    ids = [36, 0, 5, 5]
    out = torch.empty(4, 24, device=DEV)
    ops().embed_gather(table.to(DEV), torch.tensor(ids, dtype=torch.int32, device=DEV), out)
    assert np.array_equal(out.cpu().numpy(), R.embed(table, ids))
    for width in (100, 2500):
        x, w = rnd(7, width, seed=1), 1 + 0.1 * rnd(width, seed=3)
        out = torch.empty(7, width, device=DEV)
        ops().rms_norm(x.to(DEV), w.to(DEV), 1e-5, out)
        np.testing.assert_allclose(out.cpu().numpy(), R.rms_norm(x, w, 1e-5), rtol=2e-6, atol=2e-6)
    # the gate: the product's own epilogue (rows of the weight alternate gate and up)
    x, w = rnd(5, 40, seed=5), rnd(2 * 88, 40, seed=6)
    out = torch.empty(5, 88, device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out, swiglu=True)
    gu = R.gemm(x, w)
    np.testing.assert_allclose(out.cpu().numpy(), R.swiglu(gu[:, 0::2], gu[:, 1::2]), rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("H,Hk,D,rot", [(3, 1, 48, 48), (6, 3, 64, 32), (5, 1, 128, 0)])
def test_head_norm_and_rotation(H, Hk, D, rot):
    segments, page_size = [(0, 5), (37, 1), (9, 3)], 16
    tables = [[3], [4, 5, 6], [0]]
    ctx = hand_context(segments, page_size, 8, torch.float32, DEV, kv_sites={0: (Hk, D)}, tables=tables)
    T = ctx.n_tokens
    qkv = rnd(T, (H + 2 * Hk) * D, seed=D)
    qw, kw = 1 + 0.1 * rnd(D, seed=1), 1 + 0.1 * rnd(D, seed=2)
    inv = None
    if rot:
        inv = np.power(np.float32(1e6), (np.float32(-2.0) * np.arange(rot // 2, dtype=np.float32) / np.float32(rot))).astype(np.float32)
    k_cache, v_cache, table = ctx.kv(0)
    q_out = torch.empty(T, H, D, device=DEV)
    ops().qk_norm_rope_store(qkv.to(DEV), qw.to(DEV), kw.to(DEV), 1e-5, None if inv is None else torch.from_numpy(inv).to(DEV),
                             ctx.positions, ctx.row_of_token, table, page_size, q_out, k_cache, v_cache, H, Hk, D)
    positions, rows = ctx.positions.cpu().tolist(), ctx.row_of_token.cpu().tolist()
    q_ref = R.head_norm_rope(qkv[:, :H * D].reshape(T, H, D), qw, 1e-5, positions, inv)
    k_ref = R.head_norm_rope(qkv[:, H * D:(H + Hk) * D].reshape(T, Hk, D), kw, 1e-5, positions, inv)
    np.testing.assert_allclose(q_out.cpu().numpy(), q_ref, rtol=1e-5, atol=1e-5)
    for t, (pos, r) in enumerate(zip(positions, rows)):
        got = k_cache[tables[r][pos // page_size], :, pos % page_size].cpu().numpy()
        np.testing.assert_allclose(got, k_ref[t], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("H,Hk,D", [(6, 2, 48), (8, 1, 128)])
@pytest.mark.parametrize("page_size,window", [(16, None), (8, 19)])
def test_attention_over_pages(H, Hk, D, page_size, window):
    got, ref = _attention_case(H, Hk, D, page_size, window, torch.float32, attend=R.attention)
    torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-5)
    got, ref = _attention_case(H, Hk, D, 16, window, torch.bfloat16, kernel="mfma", attend=R.attention,
                               ctx_lens=(70, 1, 700, 33), q_lens=(5, 1, 1, 33))
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("width,taps", [(100, 3), (300, 4), (64, 9)])
@pytest.mark.parametrize("segments", [[(0, 1), (0, 9), (0, 2)], [(0, 40), (0, 3), (0, 1)]])
def test_short_conv_is_the_statement_bit_for_bit(width, taps, segments):
    """Few tokens take the kernel with a channel per thread, 32 or more the one with four: the same bits."""
    slots, n_tok = [3, 0, 5], sum(n for _, n in segments)
    w, bias = rnd(width, taps, seed=1, scale=0.3), rnd(width, seed=2, scale=0.1)
    state0 = rnd(8, taps - 1, width, seed=3)
    bcx = rnd(n_tok, 3 * width, seed=4)
    ctx = hand_context(segments, 16, 16, torch.float32, DEV, fixed_sites={0: (taps - 1, width)}, slots=slots)
    state = ctx.fixed_state(0)
    state.copy_(state0)
    out = torch.empty(n_tok, width, device=DEV)
    ops().short_conv(bcx.to(DEV), w.to(DEV), bias.to(DEV), state, ctx.row_of_token, ctx.seg_start, ctx.seg_len,
                     ctx.slot, out)
    at = 0
    for (_, n), slot in zip(segments, slots):
        y, s = R.short_conv(bcx[at:at + n], w, bias, state0[slot])
        assert np.array_equal(out[at:at + n].cpu().numpy(), y) and np.array_equal(state[slot].cpu().numpy(), s)
        at += n
    # rows of one token each, through the kernel that reads and shifts the history in one launch
    ctx = hand_context([(5, 1), (0, 1)], 16, 16, torch.float32, DEV, fixed_sites={0: (taps - 1, width)}, slots=[4, 1])
    state = ctx.fixed_state(0)
    state.copy_(state0)
    out = torch.empty(2, width, device=DEV)
    ops().short_conv(bcx[:2].to(DEV), w.to(DEV), bias.to(DEV), state, ctx.row_of_token, ctx.seg_start, ctx.seg_len,
                     ctx.slot, out, single_tokens=True)
    for r, slot in enumerate((4, 1)):
        y, s = R.short_conv(bcx[r:r + 1], w, bias, state0[slot])
        assert np.array_equal(out[r:r + 1].cpu().numpy(), y) and np.array_equal(state[slot].cpu().numpy(), s)


@pytest.mark.parametrize("vocab", [7, 1000, 70001])
def test_picks(vocab):
    x = rnd(6, vocab, seed=vocab)
    x[1, vocab - 1] = x[1, vocab // 2] = x[1].max() + 1
    x[2, 0] = float("nan")
    x[3] = float("nan")
    x[4] = -float("inf")
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    ops().argmax_rows(x.to(DEV), out)
    assert out.cpu().tolist() == R.argmax(x).tolist()
    n = 64
    logits = rnd(n, vocab, seed=1, scale=2.0)
    temps = torch.tensor([0.8] * (n - 2) + [0.0, 1.7])
    u = torch.rand(n, generator=torch.Generator().manual_seed(2))
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample_rows(logits.to(DEV), temps.to(DEV), u.to(DEV), out)
    want = R.sample(logits, temps, u)
    # the kernel's sums are float32, the statement's float64: a uniform within rounding of a step of
    # the CDF may fall on either side of it, so the two picks lie within 1e-5 of probability mass of
    # each other, and where the steps are far larger than that they are the same pick
    got, same = out.cpu().tolist(), 0
    for r in range(n):
        if temps[r] <= 0:
            assert got[r] == want[r]
            continue
        cdf = np.cumsum(np.exp((logits[r].double().numpy() - float(logits[r].max())) / float(temps[r])))
        assert abs(cdf[got[r]] - cdf[want[r]]) <= 1e-5 * cdf[-1], (r, got[r], want[r])
        same += got[r] == want[r]
    assert vocab > 1000 or same >= n - 4
