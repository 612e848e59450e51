"""Each kernel alone beside a plain reference, at sizes other than the
engine's: odd row counts, widths and vocabularies that are no power of two,
head sizes in steps of 16, several head/group counts, windows, short segments.
"""
import math

import numpy as np
import pytest
import torch

import plain_lfm2 as P
from gpu_helpers import hand_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from imparo_amd.kernels import ops as o
    return o


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# ---------------------------------------------------------------- GEMM
@pytest.mark.parametrize("m", [1, 5, 16, 17, 33, 64, 65, 130, 300])
@pytest.mark.parametrize("n,k", [(16, 8), (40, 96), (136, 264), (200, 1032), (1000, 64)])
def test_gemm(m, n, k):
    x, w = rnd(m, k, seed=m), rnd(n, k, seed=n + 1)
    # float32: exact products, sums of at most 1032 terms
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out)
    ref = x.double() @ w.double().t()
    assert (out.cpu().double() - ref).abs().max() <= 1e-6 * math.sqrt(k) * ref.abs().max()
    # bfloat16 operands: products are exact in float32, accumulation is float32
    xb, wb = x.to(torch.bfloat16), w.to(torch.bfloat16)
    ref = xb.double() @ wb.double().t()
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    ops().gemm(xb.to(DEV), wb.to(DEV), out)
    assert (out.cpu().double() - ref).abs().max() <= 1e-6 * math.sqrt(k) * ref.abs().max()
    outb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops().gemm(xb.to(DEV), wb.to(DEV), outb)
    assert torch.equal(outb.cpu(), out.cpu().to(torch.bfloat16))      # only the final rounding differs


def test_float32_gemm_sums_the_same_way_for_few_rows_and_many():
    """Up to 16 rows take a kernel of their own: a row's results are the same bits as in a batch of 40."""
    x, w, b = rnd(40, 1000, seed=1), rnd(210, 1000, seed=2, scale=0.3), rnd(210, seed=3)
    for swiglu in (False, True):
        many = torch.empty(40, 105 if swiglu else 210, device=DEV)
        ops().gemm(x.to(DEV), w.to(DEV), many, bias=b.to(DEV), swiglu=swiglu)
        for rows in (1, 7, 16):
            few = torch.empty(rows, many.shape[1], device=DEV)
            ops().gemm(x[:rows].to(DEV), w.to(DEV), few, bias=b.to(DEV), swiglu=swiglu)
            assert torch.equal(few, many[:rows])


@pytest.mark.parametrize("m", [1, 20, 64, 150])
def test_gemm_epilogues(m):
    """A bias, and the SwiGLU epilogue over a weight whose rows alternate gate and up, in the
    float32 kernel and both bfloat16 kernels."""
    n, k = 2 * 88, 72
    x, w, b = rnd(m, k, seed=1), rnd(n, k, seed=2, scale=0.3), rnd(n, seed=3)
    for dt in (torch.float32, torch.bfloat16):
        xd, wd = x.to(dt), w.to(dt)
        y = xd.double() @ wd.double().t() + b.double()
        out = torch.empty(m, n, device=DEV)
        ops().gemm(xd.to(DEV), wd.to(DEV), out, bias=b.to(DEV))
        torch.testing.assert_close(out.cpu().double(), y, rtol=1e-5, atol=1e-5)
        gate, up = y[:, 0::2], y[:, 1::2]
        ref = (gate / (1 + torch.exp(-gate)) * up)
        out = torch.empty(m, n // 2, device=DEV)
        ops().gemm(xd.to(DEV), wd.to(DEV), out, bias=b.to(DEV), swiglu=True)
        torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-5, atol=1e-5)
        outb = torch.empty(m, n // 2, dtype=torch.bfloat16, device=DEV)
        ops().gemm(xd.to(DEV), wd.to(DEV), outb, bias=b.to(DEV), swiglu=True)
        assert torch.equal(outb.cpu(), out.cpu().to(torch.bfloat16))
    # an odd last column never pairs with its neighbour's tile: n = 2 * odd, edge tiles
    n = 2 * 67
    w = rnd(n, k, seed=4, scale=0.3).to(torch.bfloat16)
    y = x.to(torch.bfloat16).double() @ w.double().t()
    out = torch.empty(m, n // 2, device=DEV)
    ops().gemm(x.to(torch.bfloat16).to(DEV), w.to(DEV), out, swiglu=True)
    torch.testing.assert_close(out.cpu().double(), y[:, 0::2] / (1 + torch.exp(-y[:, 0::2])) * y[:, 1::2],
                               rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("m", [1, 9, 40, 64])
def test_gemm_in_slices_of_k_and_the_norm_that_adds_them(m):
    """A few-row product over a long K may leave its result as sums over slices of K, which the
    norm that consumes it adds up in order."""
    n, k = 200, 4096 + 264
    x, w, b = rnd(m, k, seed=1).to(torch.bfloat16), rnd(n, k, seed=2, scale=0.1).to(torch.bfloat16), rnd(n, seed=3)
    slices = ops().gemm_slices(m, n, k, torch.bfloat16)
    # few weight rows: as many slices as it takes towards 256 blocks, at least 512 of K each, at most 8;
    # 8 slices of this ragged K, rounded up to chunks of 128, would leave the eighth empty: 4 then
    assert slices == 4 and ops().gemm_slices(m, n, 2048, torch.bfloat16) == 4
    assert ops().gemm_slices(m, 1024, 4608, torch.bfloat16) == 8
    assert ops().gemm_slices(m, 2048, 2048, torch.bfloat16) == (2 if m <= 16 else 4)    # 128 or 64 blocks
    assert ops().gemm_slices(m, 8192, k, torch.bfloat16) == 1       # a weight with many rows fills the chip by itself
    assert ops().gemm_slices(m, n, k, torch.float32) == 1
    # many rows and few tiles: the tile kernels take slices too, at most 4 (this K, no multiple of 128, goes to
    # the one with register staging: at least 1024 of K each; K = 2048 to the one that loads into LDS: 512)
    assert ops().gemm_slices(300, n, k, torch.bfloat16) == 4 and ops().gemm_slices(300, n, 2048, torch.bfloat16) == 4
    assert ops().gemm_slices(2048, 16384, 2048, torch.bfloat16) == 1
    x3 = rnd(300, k, seed=7).to(torch.bfloat16)
    out3 = torch.full((4, 300, n), float("nan"), device=DEV)
    ops().gemm(x3.to(DEV), w.to(DEV), out3, bias=b.to(DEV))
    torch.testing.assert_close(out3.cpu().double().sum(0), x3.double() @ w.double().t() + b.double(), rtol=1e-5, atol=1e-5)
    out = torch.full((slices, m, n), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out, bias=b.to(DEV))
    ref = x.double() @ w.double().t() + b.double()
    torch.testing.assert_close(out.cpu().double().sum(0), ref, rtol=1e-5, atol=1e-5)
    whole = torch.empty(m, n, device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), whole, bias=b.to(DEV))
    torch.testing.assert_close(out.sum(0), whole, rtol=1e-5, atol=1e-5)
    # the norm takes the slices as its delta
    res = rnd(m, n, seed=4)
    wn = 1 + 0.1 * rnd(n, seed=5)
    xd = res.to(DEV).clone()
    normed = torch.empty(m, n, device=DEV)
    ops().rms_norm(xd, wn.to(DEV), 1e-5, normed, delta=out, write_back=True)
    total = res + out.cpu().sum(0)
    torch.testing.assert_close(xd.cpu(), total, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(normed.cpu(), P.rms_norm(total, wn, 1e-5), rtol=1e-5, atol=1e-5)
    rows = torch.tensor([m - 1, 0], dtype=torch.int32, device=DEV)
    picked = torch.empty(2, n, device=DEV)
    ops().rms_norm(res.to(DEV), wn.to(DEV), 1e-5, picked, delta=out, rows=rows)
    torch.testing.assert_close(picked.cpu(), P.rms_norm(total[[m - 1, 0]], wn, 1e-5), rtol=1e-5, atol=1e-5)
    from imparo_amd.kernels import KernelArgumentError
    with pytest.raises(KernelArgumentError, match="slices"):
        ops().gemm(x.to(DEV), w.to(DEV), torch.empty(2, m, n, device=DEV))


@pytest.mark.parametrize("m", [3, 16, 24, 64])
@pytest.mark.parametrize("k", [264, 1024])
def test_gemm_with_many_weight_rows(m, k):
    """From about 12k weight rows on, few-row products go to the kernel that shares the
    activations between the waves of a block: ragged K, a last block that is cut, bias, SwiGLU."""
    n = 12288 + 2 * 37
    x, w, b = rnd(m, k, seed=1).to(torch.bfloat16), rnd(n, k, seed=2, scale=0.1).to(torch.bfloat16), rnd(n, seed=3)
    y = x.double() @ w.double().t() + b.double()
    out = torch.full((m, n), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out, bias=b.to(DEV))
    assert (out.cpu().double() - y).abs().max() <= 1e-6 * math.sqrt(k) * y.abs().max()
    act = torch.full((m, n // 2), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), act, bias=b.to(DEV), swiglu=True)
    # silu(gate) * up: an accumulation error e in gate or up shows as at most about e * max|y|
    ref = y[:, 0::2] / (1 + torch.exp(-y[:, 0::2])) * y[:, 1::2]
    assert (act.cpu().double() - ref).abs().max() <= 1e-6 * math.sqrt(k) * y.abs().max() * max(1.0, y.abs().max().item())


@pytest.mark.parametrize("m,n,k,tile", [(2600, 3900, 256, 0), (2600, 3904, 1152, 0), (3900, 4002, 384, 0),
                                        (1500, 3900, 640, 0), (2600, 3904, 200, 0), (70, 100, 128, 0),
                                        (700, 1000, 384, 258), (700, 1000, 384, 262), (700, 1000, 384, 263),
                                        (700, 1000, 384, 358), (700, 1000, 384, 352),
                                        (700, 1000, 256, 452), (700, 1000, 1280, 452), (130, 250, 2048, 452),
                                        (700, 1000, 384, 351), (100, 250, 2048, 451), (128, 1000, 512, 451),
                                        (128, 16384, 2048, 0), (96, 2048, 8192, 0), (65, 3072, 2048, 0)])
def test_gemm_with_large_tiles(m, n, k, tile):
    """Many rows: K a multiple of 128 goes to the kernel that loads straight into LDS, with a tile
    of 256 or 128 rows by 256, 192, 128 or 64 weight rows, whichever its plan finds fastest (`tile`
    other than 0 names one, an argument of the entry point for tests and measurements, so that each is met);
    another K to the tile kernels with register staging. Edges in both directions, an odd number
    of column pairs, a bias, both epilogues and output types."""
    _large_tile_case(m, n, k, tile)


def _large_tile_case(m, n, k, variant=0):
    x, w, b = rnd(m, k, seed=1, scale=0.5).to(torch.bfloat16), rnd(n, k, seed=2, scale=0.3).to(torch.bfloat16), rnd(n, seed=3)
    y = x.float() @ w.float().t() + b                       # float32 on the CPU: products exact, sums to 1e-6 sqrt(k)
    bound = 1e-6 * math.sqrt(k) * float(y.abs().max())
    out = torch.full((m, n), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out, bias=b.to(DEV), variant=variant)
    assert (out.cpu() - y).abs().max() <= 4 * bound
    outb = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), outb, bias=b.to(DEV), variant=variant)
    assert torch.equal(outb.cpu(), out.cpu().to(torch.bfloat16))
    ref = torch.nn.functional.silu(y[:, 0::2].double()) * y[:, 1::2].double()
    out = torch.full((m, n // 2), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out, bias=b.to(DEV), swiglu=True, variant=variant)
    torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-5, atol=8 * bound)
    outb = torch.full((m, n // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), outb, bias=b.to(DEV), swiglu=True, variant=variant)
    assert torch.equal(outb.cpu(), out.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("m,n,k", [(700, 1000, 384), (2048, 2048, 2048), (130, 250, 1024), (1500, 3902, 640)])
def test_gemm_added_to_what_the_output_holds(m, n, k):
    """The epilogue that adds: bit for bit what adding the plain product afterwards gives, at the
    tiles' edges too; refused where the tile kernel does not run the product."""
    from imparo_amd.kernels import KernelArgumentError
    x, w, b = rnd(m, k, seed=1, scale=0.5).to(torch.bfloat16), rnd(n, k, seed=2, scale=0.3).to(torch.bfloat16), rnd(n, seed=3)
    assert ops().gemm_adds(m, n, k, torch.bfloat16)
    held = rnd(m, n, seed=4).to(DEV)
    plain = torch.full((m, n), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), plain, bias=b.to(DEV)) if ops().gemm_slices(m, n, k, torch.bfloat16) == 1 else None
    out = held.clone()
    ops().gemm(x.to(DEV), w.to(DEV), out, bias=b.to(DEV), add=True)
    y = x.float() @ w.float().t() + b
    assert (out.cpu() - (held.cpu() + y)).abs().max() <= 4e-6 * math.sqrt(k) * float(y.abs().max())
    if ops().gemm_slices(m, n, k, torch.bfloat16) == 1:
        assert torch.equal(out, held + plain)
    with pytest.raises(KernelArgumentError, match="cannot be added"):
        ops().gemm(x[:8].to(DEV), w.to(DEV), held[:8].clone(), add=True)
    with pytest.raises(KernelArgumentError, match="cannot be added"):
        ops().gemm(x.to(DEV), w.to(DEV), torch.empty(m, n, dtype=torch.bfloat16, device=DEV), add=True)


@pytest.mark.parametrize("m,n,k,slices", [(1000, 2000, 8192, 2), (500, 2000, 8192, 4), (4000, 2000, 8192, 2),
                                          (300, 2000, 4096, 4)])
def test_gemm_with_large_tiles_in_slices_of_k(m, n, k, slices):
    """Few tiles and a long K: slices of K on the large tiles, as many as the plan's model of the time finds
    fastest (on two stages or on four)."""
    assert ops().gemm_slices(m, n, k, torch.bfloat16) == slices
    x, w, b = rnd(m, k, seed=1, scale=0.5).to(torch.bfloat16), rnd(n, k, seed=2, scale=0.3).to(torch.bfloat16), rnd(n, seed=3)
    y = x.float() @ w.float().t() + b
    out = torch.full((slices, m, n), float("nan"), device=DEV)
    ops().gemm(x.to(DEV), w.to(DEV), out, bias=b.to(DEV))
    assert (out.cpu().sum(0) - y).abs().max() <= 4e-6 * math.sqrt(k) * float(y.abs().max())
    # each slice is its own range of K; the bias rides on the first
    per = k // slices
    part = x[:, per:2 * per].float() @ w[:, per:2 * per].float().t()
    assert (out[1].cpu() - part).abs().max() <= 4e-6 * math.sqrt(per) * float(part.abs().max())


def test_gemm_refuses_what_it_cannot_take():
    from imparo_amd.kernels import KernelArgumentError
    x, w = rnd(4, 12).to(torch.bfloat16).to(DEV), rnd(8, 12).to(torch.bfloat16).to(DEV)
    with pytest.raises(KernelArgumentError, match="multiple of 8"):
        ops().gemm(x, w, torch.empty(4, 8, dtype=torch.float32, device=DEV))
    with pytest.raises(KernelArgumentError, match="columns"):
        ops().gemm(rnd(4, 16).to(DEV), rnd(8, 24).to(DEV), torch.empty(4, 8, device=DEV))
    with pytest.raises(KernelArgumentError, match="GPU only"):
        ops().gemm(rnd(4, 16), rnd(8, 16), torch.empty(4, 8))
    # float32 takes any inner size
    out = torch.empty(3, 5, device=DEV)
    ops().gemm(rnd(3, 7).to(DEV), rnd(5, 7, seed=1).to(DEV), out)
    torch.testing.assert_close(out.cpu(), rnd(3, 7) @ rnd(5, 7, seed=1).t(), rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- rows
@pytest.mark.parametrize("width", [16, 100, 2048, 2500])
def test_rms_norm(width):
    x, d, w = rnd(7, width, seed=1), rnd(7, width, seed=2), 1 + 0.1 * rnd(width, seed=3)
    for eps in (1e-5, 1e-2):
        out = torch.empty(7, width, device=DEV)
        ops().rms_norm(x.to(DEV), w.to(DEV), eps, out)
        torch.testing.assert_close(out.cpu(), P.rms_norm(x, w, eps), rtol=2e-6, atol=2e-6)
    # fused add, written back
    xd = x.to(DEV).clone()
    out = torch.empty(7, width, dtype=torch.bfloat16, device=DEV)
    ops().rms_norm(xd, w.to(DEV), 1e-5, out, delta=d.to(DEV), write_back=True)
    assert torch.equal(xd.cpu(), x + d)
    ref = P.rms_norm(x + d, w, 1e-5)
    assert (out.cpu().float() - ref).abs().max() <= 2 ** -8 * ref.abs().max()
    # selected rows, with a delta, nothing written back
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    xd = x.to(DEV).clone()
    out = torch.empty(3, width, device=DEV)
    ops().rms_norm(xd, w.to(DEV), 1e-5, out, delta=d.to(DEV), rows=rows)
    assert torch.equal(xd.cpu(), x)
    torch.testing.assert_close(out.cpu(), P.rms_norm((x + d)[[5, 0, 5]], w, 1e-5), rtol=2e-6, atol=2e-6)


def test_embed_gather():
    table = rnd(37, 24, seed=4)
    ids = torch.tensor([36, 0, 5, 5], dtype=torch.int32, device=DEV)
    for t in (table, table.to(torch.bfloat16)):
        out = torch.empty(4, 24, device=DEV)
        ops().embed_gather(t.to(DEV), ids, out)
        assert torch.equal(out.cpu(), t.float()[[36, 0, 5, 5]])


def test_fill_sites_sets_one_slot_of_every_site():
    sites = [torch.full((5, 2, 8), 7.0, device=DEV), torch.full((5, 3), 7.0, device=DEV),
             torch.full((5, 4000), 7.0, device=DEV)]
    base = torch.tensor([t.data_ptr() for t in sites], dtype=torch.int64, device=DEV)
    per_slot = torch.tensor([t[0].numel() for t in sites], dtype=torch.int64, device=DEV)
    value = torch.tensor([0.0, -1.5, 2.0], device=DEV)
    ops().fill_sites(base, per_slot, value, 3)
    for t, v in zip(sites, (0.0, -1.5, 2.0)):
        assert bool((t[3] == v).all()) and bool((t[[0, 1, 2, 4]] == 7.0).all())


# ---------------------------------------------------------------- norm + rotation + cache write
@pytest.mark.parametrize("H,Hk,D,rot", [(4, 2, 16, 16), (3, 1, 48, 48), (6, 3, 64, 32), (2, 2, 80, 80), (5, 1, 128, 0)])
@pytest.mark.parametrize("page_size,vt", [(4, False), (16, False), (16, True)])
def test_qk_norm_rope_store(H, Hk, D, rot, page_size, vt):
    segments = [(0, 5), (37, 1), (9, 3)]
    tables = [[3, 1], list(range(4, 4 + 40 // page_size + 1)), [0, 2, 14][: (12 + page_size - 1) // page_size]]
    n_pages = 16
    for dtype in (torch.float32, torch.bfloat16):
        ctx = hand_context(segments, page_size, n_pages, dtype, DEV, kv_sites={0: (Hk, D)}, tables=tables,
                           v_transposed=vt)
        T = ctx.n_tokens
        qkv = rnd(T, (H + 2 * Hk) * D, seed=D)
        qw, kw = 1 + 0.1 * rnd(D, seed=1), 1 + 0.1 * rnd(D, seed=2)
        base = 10000.0
        inv = None
        if rot:
            i = np.arange(rot // 2, dtype=np.float32)
            inv = torch.from_numpy(np.power(np.float32(base), (np.float32(-2.0) * i / np.float32(rot))).astype(np.float32)).to(DEV)
        k_cache, v_cache, table = ctx.kv(0)
        q_out = torch.empty(T, H, D, dtype=dtype, device=DEV)
        ops().qk_norm_rope_store(qkv.to(DEV), qw.to(DEV), kw.to(DEV), 1e-5, inv, ctx.positions, ctx.row_of_token,
                                 table, page_size, q_out, k_cache, v_cache, H, Hk, D, v_transposed=vt)
        if vt:
            v_cache = v_cache.transpose(2, 3)           # viewed [page, kv head, slot, dim] again
        positions = ctx.positions.cpu().tolist()
        q = qkv[:, :H * D].reshape(T, H, D)
        k = qkv[:, H * D:(H + Hk) * D].reshape(T, Hk, D)
        v = qkv[:, (H + Hk) * D:].reshape(T, Hk, D)
        q_ref, k_ref = P.rms_norm(q, qw, 1e-5), P.rms_norm(k, kw, 1e-5)
        if rot:
            q_ref, k_ref = P.rope_neox(q_ref, positions, base, rot), P.rope_neox(k_ref, positions, base, rot)
        tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
        torch.testing.assert_close(q_out.cpu().float(), q_ref, **tol)
        rows = ctx.row_of_token.cpu().tolist()
        written = torch.zeros(n_pages, page_size, dtype=torch.bool)
        for t, (pos, r) in enumerate(zip(positions, rows)):
            page = tables[r][pos // page_size]
            written[page, pos % page_size] = True
            torch.testing.assert_close(k_cache[page, :, pos % page_size].cpu().float(), k_ref[t], **tol)
            torch.testing.assert_close(v_cache[page, :, pos % page_size].cpu().float(), v[t], **tol)
        # nothing else was touched
        untouched = ~written
        assert k_cache.cpu().float().permute(0, 2, 1, 3)[untouched].abs().sum() == 0
        assert v_cache.cpu().float().permute(0, 2, 1, 3)[untouched].abs().sum() == 0


@pytest.mark.parametrize("H,Hk,D,rot", [(4, 2, 16, 16), (5, 1, 64, 64), (32, 8, 64, 64), (9, 3, 64, 32), (6, 3, 96, 32),
                                        (3, 1, 144, 144), (2, 2, 272, 0)])
@pytest.mark.parametrize("vt", [False, True])
def test_qk_norm_rope_store_many_tokens(H, Hk, D, rot, vt):
    """From 96 tokens on a launch takes the kernel with a block per token. A token's results are the
    same bits whichever kernel it met (the same tokens again, a few at a time), and right."""
    segments, page_size, n_pages = [(0, 270), (5, 141)], 16, 30
    tables = [[3, 1, 7, 9, 11, 29, 28, 13, 15, 17, 19, 21, 23, 25, 27, 5, 6], [0, 2, 4, 8, 10, 12, 14, 16, 18, 20]]
    for dtype in (torch.float32, torch.bfloat16):
        qkv = rnd(411, (H + 2 * Hk) * D, seed=D).to(DEV)
        qw, kw = (1 + 0.1 * rnd(D, seed=1)).to(DEV), (1 + 0.1 * rnd(D, seed=2)).to(DEV)
        inv = None
        if rot:
            i = np.arange(rot // 2, dtype=np.float32)
            inv = torch.from_numpy(np.power(np.float32(1e6), (np.float32(-2.0) * i / np.float32(rot))).astype(np.float32)).to(DEV)
        results = []
        for step in (411, 7):
            ctx = hand_context(segments, page_size, n_pages, dtype, DEV, kv_sites={0: (Hk, D)}, tables=tables,
                               v_transposed=vt)
            k_cache, v_cache, table = ctx.kv(0)
            q_out = torch.empty(411, H, D, dtype=dtype, device=DEV)
            for t0 in range(0, 411, step):
                t1 = min(411, t0 + step)
                ops().qk_norm_rope_store(qkv[t0:t1], qw, kw, 1e-6, inv, ctx.positions[t0:t1], ctx.row_of_token[t0:t1],
                                         table, page_size, q_out[t0:t1], k_cache, v_cache, H, Hk, D, v_transposed=vt)
            results.append((q_out.cpu(), k_cache.cpu().clone(), v_cache.cpu().clone()))
        for a, b in zip(*results):
            assert torch.equal(a, b)
        positions = ctx.positions.cpu().tolist()
        q = qkv.cpu()[:, :H * D].reshape(411, H, D)
        q_ref = P.rms_norm(q, qw.cpu(), 1e-6)
        if rot:
            q_ref = P.rope_neox(q_ref, positions, 1e6, rot)
        tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
        torch.testing.assert_close(results[0][0].float(), q_ref, **tol)
        k = qkv.cpu()[:, H * D:(H + Hk) * D].reshape(411, Hk, D)
        k_ref = P.rms_norm(k, kw.cpu(), 1e-6)
        if rot:
            k_ref = P.rope_neox(k_ref, positions, 1e6, rot)
        v = qkv.cpu()[:, (H + Hk) * D:].reshape(411, Hk, D)
        kc, vc = results[0][1].float(), results[0][2].float()
        if vt:
            vc = vc.transpose(2, 3)
        for t, (pos, r) in enumerate(zip(positions, ctx.row_of_token.cpu().tolist())):
            page = tables[r][pos // page_size]
            torch.testing.assert_close(kc[page, :, pos % page_size], k_ref[t], **tol)
            torch.testing.assert_close(vc[page, :, pos % page_size], v[t], **tol)


@pytest.mark.parametrize("n_tokens", [5, 450])
def test_rotation_at_far_positions(n_tokens):
    """Angles of 1e5 radians and more (positions up to 127,999, a base of 10 so that the slow pairs turn
    too): sines and cosines keep float32 accuracy after the argument's reduction. A wrong multiple of
    pi/2, or a quarter turn taken the wrong way, would show as errors of order one."""
    H, Hk, D = 3, 1, 64
    g = torch.Generator().manual_seed(5)
    positions = torch.randint(90000, 128000, (n_tokens,), generator=g).to(torch.int32)
    positions[0], positions[1] = 127999, 0
    qkv = rnd(n_tokens, (H + 2 * Hk) * D, seed=9)
    i = np.arange(D // 2, dtype=np.float32)
    inv_np = np.power(np.float32(10.0), (np.float32(-2.0) * i / np.float32(D))).astype(np.float32)
    q_out = torch.empty(n_tokens, H, D, device=DEV)
    ops().qk_norm_rope_store(qkv.to(DEV), None, None, 1e-6, torch.from_numpy(inv_np).to(DEV), positions.to(DEV),
                             torch.zeros(n_tokens, dtype=torch.int32, device=DEV), None, 16, q_out, None, None, H, Hk, D)
    theta = (positions.numpy().astype(np.float64)[:, None] * inv_np.astype(np.float64)).astype(np.float32).astype(np.float64)
    cos, sin = torch.from_numpy(np.cos(theta)).unsqueeze(1), torch.from_numpy(np.sin(theta)).unsqueeze(1)
    x = qkv[:, :H * D].reshape(n_tokens, H, D).double()
    ref = torch.cat([x[..., :32] * cos - x[..., 32:] * sin, x[..., :32] * sin + x[..., 32:] * cos], dim=-1)
    assert theta.max() > 1e5
    torch.testing.assert_close(q_out.cpu().double(), ref, rtol=0, atol=2e-6)


@pytest.mark.parametrize("H,Hk,D", [(7, 2, 64), (3, 1, 32)])
def test_rotation_of_neighbouring_pairs_many_tokens(H, Hk, D):
    """Pairs (2i, 2i + 1) instead of (i, i + half): the kernel with a block per token (heads of 64 take
    four elements a lane there) gives the bits of the kernel with a wave per head, and the rotation
    is the one written out here."""
    segments, page_size, n_pages = [(3, 411)], 16, 30
    qkv = rnd(411, (H + 2 * Hk) * D, seed=D + 1).to(DEV)
    qw, kw = (1 + 0.1 * rnd(D, seed=1)).to(DEV), (1 + 0.1 * rnd(D, seed=2)).to(DEV)
    i = np.arange(D // 2, dtype=np.float32)
    inv_np = np.power(np.float32(1e4), (np.float32(-2.0) * i / np.float32(D))).astype(np.float32)
    inv = torch.from_numpy(inv_np).to(DEV)
    results = []
    for step in (411, 9):
        ctx = hand_context(segments, page_size, n_pages, torch.float32, DEV, kv_sites={0: (Hk, D)})
        k_cache, v_cache, table = ctx.kv(0)
        q_out = torch.empty(411, H, D, device=DEV)
        for t0 in range(0, 411, step):
            t1 = min(411, t0 + step)
            ops().qk_norm_rope_store(qkv[t0:t1], qw, kw, 1e-6, inv, ctx.positions[t0:t1], ctx.row_of_token[t0:t1],
                                     table, page_size, q_out[t0:t1], k_cache, v_cache, H, Hk, D, interleaved=True)
        results.append((q_out.cpu(), k_cache.cpu().clone(), v_cache.cpu().clone()))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    positions = np.asarray(ctx.positions.cpu().tolist(), dtype=np.float64)
    theta = torch.from_numpy((positions[:, None] * inv_np.astype(np.float64)).astype(np.float32))
    cos, sin = theta.cos().unsqueeze(1), theta.sin().unsqueeze(1)
    x = P.rms_norm(qkv.cpu()[:, :H * D].reshape(411, H, D), qw.cpu(), 1e-6)
    ref = x.clone()
    ref[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
    ref[..., 1::2] = x[..., 0::2] * sin + x[..., 1::2] * cos
    torch.testing.assert_close(results[0][0], ref, rtol=1e-5, atol=1e-5)
    assert (ref - x).abs().max() > 0.5          # it did turn


# ---------------------------------------------------------------- attention
def _attention_case(H, Hk, D, page_size, window, dtype, sharpen=None, seed=0, kernel="wave", v_transposed=None,
                    ctx_lens=(70, 1, 200, 33), q_lens=(5, 1, 1, 33), attend=P.attend, table_width=0, prefill_splits=1):
    """Rows at different depths of their contexts; the cache is filled by hand
    from whole-sequence k, v; the reference attends over the whole sequences."""
    # the last q_len positions of each context are queried
    vt = (kernel == "mfma") if v_transposed is None else v_transposed
    n_pages = sum((c + page_size - 1) // page_size for c in ctx_lens) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    tables, nxt = [], 0
    for c in ctx_lens:
        k = (c + page_size - 1) // page_size
        tables.append(perm[nxt:nxt + k])
        nxt += k
    if table_width:                            # room for longer contexts: entries nobody may read (their pages hold NaN)
        tables[0] = tables[0] + perm[nxt:nxt + 3] * ((table_width - len(tables[0]) + 2) // 3)
    segments = [(c - ql, ql) for c, ql in zip(ctx_lens, q_lens)]
    ctx = hand_context(segments, page_size, n_pages, dtype, DEV, kv_sites={0: (Hk, D)}, tables=tables,
                       v_transposed=vt)
    k_cache, v_cache, table = ctx.kv(0)
    k_cache.fill_(float("nan"))                # a key read from outside the context poisons the output
    v_cache.fill_(float("nan"))
    qs, refs = [], []
    for r, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
        q, k, v = rnd(c, H, D, seed=seed + 10 * r), rnd(c, Hk, D, seed=seed + 10 * r + 1), rnd(c, Hk, D, seed=seed + 10 * r + 2)
        if sharpen is not None:                # one far key stands out for the last query
            far = sharpen(c)
            k[far] = 0
            k[far, :, 0] = 12.0
            q[-1] = 0
            q[-1, :, 0] = 12.0
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
        for p in range(c):
            page = tables[r][p // page_size]
            k_cache[page, :, p % page_size] = k[p].to(dtype).to(DEV)
            if vt:
                v_cache[page, :, :, p % page_size] = v[p].to(dtype).to(DEV)
            else:
                v_cache[page, :, p % page_size] = v[p].to(dtype).to(DEV)
        ref = torch.as_tensor(attend(q, k, v, range(c), 1.0 / math.sqrt(D), window))
        qs.append(q[c - ql:])
        refs.append(ref[c - ql:])
    q_all = torch.cat(qs).to(dtype).to(DEV)
    out = torch.full((ctx.n_tokens, H * D), float("nan"), dtype=dtype, device=DEV)
    scale = 1.0 / math.sqrt(D)
    if kernel == "wave":
        ops().attention(q_all, k_cache, v_cache, out, ctx.positions, ctx.row_of_token, table, scale, window,
                        v_transposed=vt)
    else:
        n_splits = (ctx.max_context + 255) // 256
        part_o = torch.full((ctx.n_single_rows * H * n_splits * D,), float("nan"), device=DEV)
        part_ml = torch.full((ctx.n_single_rows * H * n_splits * 2,), float("nan"), device=DEV)
        ops().attention_decode(q_all, k_cache, v_cache, out, part_o, part_ml, ctx.single_rows, ctx.n_single_rows,
                               ctx.seg_start, ctx.positions, table, scale, window, ctx.max_context)
        parts_o = parts_ml = None
        if prefill_splits > 1:                 # NaN where no part writes: a part without keys must not be read
            parts_o = torch.full((ctx.n_tokens, H, prefill_splits, D), float("nan"), device=DEV)
            parts_ml = torch.full((ctx.n_tokens, H, prefill_splits, 2), float("nan"), device=DEV)
        ops().attention_prefill(q_all, k_cache, v_cache, out, ctx.portion_rows, ctx.n_portion_rows,
                                sum((n + 63) // 64 for n in ctx.host_seg_len if n > 1), ctx.seg_start, ctx.seg_len, ctx.positions, table, scale, window,
                                parts_o, parts_ml, prefill_splits)
    return out.cpu().float().reshape(-1, H, D), torch.cat(refs)


@pytest.mark.parametrize("H,Hk,D", [(1, 1, 16), (6, 2, 48), (5, 5, 64), (8, 1, 128), (4, 2, 80)])
@pytest.mark.parametrize("page_size,window", [(4, None), (16, None), (64, None), (8, 19), (16, 64), (4, 1)])
def test_attention(H, Hk, D, page_size, window):
    got, ref = _attention_case(H, Hk, D, page_size, window, torch.float32)
    torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-5)
    got, ref = _attention_case(H, Hk, D, page_size, window, torch.bfloat16)
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)      # one rounding of the output, P in float32


@pytest.mark.parametrize("H,Hk,D", [(32, 8, 64), (24, 8, 48), (28, 4, 32), (9, 3, 80)])
def test_matrix_core_attention_grids_of_any_width(H, Hk, D):
    """Sixteen fresh prompts in one launch: more than 256 blocks, in rows of the grid whose width
    does not divide 256. Every (tile, head) must be taken exactly once however the blocks are
    ordered (an output nobody wrote stays NaN)."""
    lens = (64, 63, 1, 47, 38, 23, 70, 85, 36, 15, 4, 32, 50, 54, 33, 65)
    got, ref = _attention_case(H, Hk, D, 64, None, torch.bfloat16, kernel="mfma", ctx_lens=lens, q_lens=lens)
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)
    lens = (300, 1, 129, 77, 191)                 # several tiles a row
    got, ref = _attention_case(H, Hk, D, 16, 100, torch.bfloat16, kernel="mfma", ctx_lens=lens, q_lens=lens)
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,Hk,D", [(1, 1, 16), (6, 2, 48), (5, 5, 64), (8, 1, 128), (4, 2, 80), (40, 2, 32),
                                    (6, 3, 64), (12, 3, 96)])
@pytest.mark.parametrize("page_size,window", [(16, None), (64, None), (32, 19), (16, 64), (16, 1), (128, 300)])
def test_matrix_core_attention(H, Hk, D, page_size, window):
    """The split-KV decode kernel and the tiled prefill kernel: contexts that
    span several splits of 256 keys and several tiles of 64 queries."""
    got, ref = _attention_case(H, Hk, D, page_size, window, torch.bfloat16, kernel="mfma",
                               ctx_lens=(70, 1, 700, 33, 300, 513, 256), q_lens=(5, 1, 1, 33, 150, 1, 1))
    # attention weights are rounded to bfloat16 before the second product: 2^-9 relative each
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)
    # and the general kernel reads the transposed layout too
    got, ref = _attention_case(H, Hk, D, page_size, window, torch.bfloat16, kernel="wave", v_transposed=True)
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,Hk,D,window", [(8, 2, 64, None), (4, 1, 128, None), (6, 2, 48, None), (8, 2, 64, 9000)])
def test_decode_attention_over_many_splits(H, Hk, D, window):
    """Single tokens deep in long contexts: 79, 65, 33 and 2 splits of 256 keys meet in the merge, which takes
    several splits side by side and in groups (more than one group, more than one round of 64 splits, an
    odd remainder). One far key stands out for every query, so a split lost or weighed wrongly shows."""
    page_size, ctx_lens = 64, (20001, 16385, 8200, 300)
    tables, nxt = [], 0
    for c in ctx_lens:
        n = (c + page_size - 1) // page_size
        tables.append(list(range(nxt, nxt + n)))
        nxt += n
    ctx = hand_context([(c - 1, 1) for c in ctx_lens], page_size, nxt, torch.bfloat16, DEV, kv_sites={0: (Hk, D)},
                       tables=tables, v_transposed=True)
    k_cache, v_cache, table = ctx.kv(0)
    qs, refs = [], []
    scale = 1.0 / math.sqrt(D)
    for r, c in enumerate(ctx_lens):
        q, k, v = rnd(1, H, D, seed=50 + r), rnd(c, Hk, D, seed=60 + r), rnd(c, Hk, D, seed=70 + r)
        far = 700 * (r + 1) % c if window is None else max(0, c - window) + 3 * r        # (near the window's far end)
        k[far] = 0
        k[far, :, 0] = 6.0
        q[0, :, 0] = 6.0 / scale / 6.0 * 1.5            # the far key's score stands 9 above the others' spread
        q, k, v = (t.to(torch.bfloat16).float() for t in (q, k, v))
        pages = len(tables[r])
        kp = torch.zeros(pages * page_size, Hk, D); kp[:c] = k
        vp = torch.zeros(pages * page_size, Hk, D); vp[:c] = v
        k_cache[tables[r]] = kp.reshape(pages, page_size, Hk, D).permute(0, 2, 1, 3).to(torch.bfloat16).to(DEV)
        v_cache[tables[r]] = vp.reshape(pages, page_size, Hk, D).permute(0, 2, 3, 1).to(torch.bfloat16).to(DEV)
        lo = 0 if window is None else max(0, c - window)
        kk, vv = k[lo:].repeat_interleave(H // Hk, dim=1), v[lo:].repeat_interleave(H // Hk, dim=1)
        w = torch.softmax(torch.einsum("hd,chd->hc", q[0].double(), kk.double()) * scale, dim=-1)
        refs.append(torch.einsum("hc,chd->hd", w, vv.double()).float())
        qs.append(q)
    q_all = torch.cat(qs).to(torch.bfloat16).to(DEV)
    out = torch.full((ctx.n_tokens, H * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    n_splits = (ctx.max_context + 255) // 256
    part_o = torch.full((ctx.n_single_rows * H * n_splits * D,), float("nan"), device=DEV)
    part_ml = torch.full((ctx.n_single_rows * H * n_splits * 2,), float("nan"), device=DEV)
    ops().attention_decode(q_all, k_cache, v_cache, out, part_o, part_ml, ctx.single_rows, ctx.n_single_rows,
                           ctx.seg_start, ctx.positions, table, scale, window, ctx.max_context)
    torch.testing.assert_close(out.cpu().float().reshape(-1, H, D), torch.stack(refs), rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,Hk,D", [(6, 3, 64), (40, 2, 32), (12, 3, 96), (8, 1, 128)])
@pytest.mark.parametrize("page_size,window", [(16, None), (32, 19), (128, 300)])
@pytest.mark.parametrize("parts", [2, 3, 8])
def test_matrix_core_attention_with_the_keys_in_parts(H, Hk, D, page_size, window, parts):
    """Prompt portions whose blocks walk their keys in parts, merged by a second launch (few queries
    over long contexts); short contexts leave some parts without keys."""
    got, ref = _attention_case(H, Hk, D, page_size, window, torch.bfloat16, kernel="mfma", prefill_splits=parts,
                               ctx_lens=(70, 1, 700, 33, 300, 513, 256), q_lens=(5, 1, 1, 33, 150, 1, 1))
    torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)
    assert ops().attention_prefill_splits(8, 16, 8, 64, 30000) == 8          # 128 blocks: eight parts make 1024
    assert ops().attention_prefill_splits(8, 16, 8, 64, 3000) == 2           # at least 1024 keys to a part
    assert ops().attention_prefill_splits(8, 16, 8, 64, 1500) == 1           # a short context is walked whole
    assert ops().attention_prefill_splits(32, 16, 8, 64, 30000) == 2         # 512 blocks
    assert ops().attention_prefill_splits(32, 32, 8, 64, 30000) == 3         # 512 blocks of 32 queries a wave: two rounds of 768
    assert ops().attention_prefill_splits(32, 32, 8, 64, 9000) == 1          # ... over a long context only
    assert ops().attention_prefill_splits(64, 32, 8, 64, 30000) == 2         # 1,024 such blocks
    assert ops().attention_prefill_splits(128, 32, 8, 64, 30000) == 1        # 2,048: enough
    assert ops().attention_prefill_splits(8, 16, 8, 80, 30000) == 1          # (the kernel for other head sizes has none)


@pytest.mark.parametrize("H,Hk,D,ctx,q", [(64, 16, 32, 1100, 1024), (32, 8, 64, 2100, 2048)])
def test_matrix_core_attention_with_32_queries_a_wave(H, Hk, D, ctx, q):
    """Many query tiles and heads, and block tables with room for 8,192 positions: the prompt kernel
    then gives each wave 32 queries. The same rows with narrow tables (16 queries a wave) agree."""
    wide, ref = _attention_case(H, Hk, D, 64, None, torch.bfloat16, kernel="mfma", ctx_lens=(ctx, 40), q_lens=(q, 1),
                                table_width=130)
    torch.testing.assert_close(wide, ref, rtol=2 ** -6, atol=2 ** -6)
    narrow, _ = _attention_case(H, Hk, D, 64, None, torch.bfloat16, kernel="mfma", ctx_lens=(ctx, 40), q_lens=(q, 1))
    torch.testing.assert_close(wide, narrow, rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.parametrize("H,Hk,D", [(8, 2, 64), (5, 5, 64), (40, 2, 64), (4, 1, 128)])
@pytest.mark.parametrize("page_size,window,interleaved,normed,rotated", [
    (16, None, False, True, True), (64, None, False, True, True), (64, 100, True, True, True),
    (32, 1, False, True, True), (16, None, False, False, True), (64, 300, False, True, False)])
def test_decode_attention_from_the_projection_rows(H, Hk, D, page_size, window, interleaved, normed, rotated):
    """Rows of one token whose keys and values are not in the cache yet: one launch norms and rotates
    q and k, attends over the cached keys and the new one, and writes the new key and value into their
    page. Held to the plain functions, and to the two launches it replaces. The new position's slot
    holds NaN beforehand (so does every slot beyond the contexts): reading it before it is written,
    or instead of the registers, would poison the output."""
    ctx_lens = (1, 70, 256, 257, 700, 513, 33, 512)
    n_pages = sum((c + page_size - 1) // page_size for c in ctx_lens) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(3)).tolist()
    tables, nxt = [], 0
    for c in ctx_lens:
        k = (c + page_size - 1) // page_size
        tables.append(perm[nxt:nxt + k])
        nxt += k
    ctx = hand_context([(c - 1, 1) for c in ctx_lens], page_size, n_pages, torch.bfloat16, DEV, kv_sites={0: (Hk, D)},
                       tables=tables, v_transposed=True)
    k_cache, v_cache, table = ctx.kv(0)
    k_cache.fill_(float("nan"))
    v_cache.fill_(float("nan"))
    R = len(ctx_lens)
    qkv = rnd(R, (H + 2 * Hk) * D, seed=11)
    qw, kw = 1 + 0.1 * rnd(D, seed=1), 1 + 0.1 * rnd(D, seed=2)
    base = 1e4
    i = np.arange(D // 2, dtype=np.float32)
    inv_np = np.power(np.float32(base), (np.float32(-2.0) * i / np.float32(D))).astype(np.float32)

    def turned(x, pos, weight):              # x [heads, D] at one position
        if normed:
            x = P.rms_norm(x, weight, 1e-5)
        if not rotated:
            return x
        theta = torch.from_numpy((np.float64(pos) * inv_np.astype(np.float64)).astype(np.float32))
        cos, sin = theta.cos(), theta.sin()
        out = x.clone()
        if interleaved:
            out[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
            out[..., 1::2] = x[..., 0::2] * sin + x[..., 1::2] * cos
        else:
            h = D // 2
            out[..., :h] = x[..., :h] * cos - x[..., h:] * sin
            out[..., h:] = x[..., :h] * sin + x[..., h:] * cos
        return out

    bf = lambda t: t.to(torch.bfloat16).float()
    refs, new_k, new_v = [], [], []
    for r, c in enumerate(ctx_lens):
        k, v = bf(rnd(c, Hk, D, seed=20 + r)), bf(rnd(c, Hk, D, seed=40 + r))
        for p in range(c - 1):
            page = tables[r][p // page_size]
            k_cache[page, :, p % page_size] = k[p].to(torch.bfloat16).to(DEV)
            v_cache[page, :, :, p % page_size] = v[p].to(torch.bfloat16).to(DEV)
        q_r = qkv[r, :H * D].reshape(H, D)
        k[c - 1] = bf(turned(qkv[r, H * D:(H + Hk) * D].reshape(Hk, D), c - 1, kw))
        v[c - 1] = bf(qkv[r, (H + Hk) * D:].reshape(Hk, D))
        q = torch.zeros(c, H, D)
        q[c - 1] = bf(turned(q_r, c - 1, qw))
        refs.append(torch.as_tensor(P.attend(q, k, v, range(c), 1.0 / math.sqrt(D), window))[c - 1])
        new_k.append(k[c - 1])
        new_v.append(v[c - 1])
    ref = torch.stack(refs)
    scale = 1.0 / math.sqrt(D)
    n_splits = (ctx.max_context + 255) // 256
    qw_d, kw_d = (qw.to(DEV), kw.to(DEV)) if normed else (None, None)
    inv_d = torch.from_numpy(inv_np).to(DEV) if rotated else None
    # the two launches, on a copy of the caches
    k2, v2 = k_cache.clone(), v_cache.clone()
    q2 = torch.empty(R, H, D, dtype=torch.bfloat16, device=DEV)
    ops().qk_norm_rope_store(qkv.to(DEV), qw_d, kw_d, 1e-5, inv_d, ctx.positions, ctx.row_of_token, table, page_size,
                             q2, k2, v2, H, Hk, D, v_transposed=True, interleaved=interleaved)
    two = torch.full((R, H * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    part_o = torch.full((R * H * n_splits * D,), float("nan"), device=DEV)
    part_ml = torch.full((R * H * n_splits * 2,), float("nan"), device=DEV)
    ops().attention_decode(q2, k2, v2, two, part_o, part_ml, ctx.single_rows, ctx.n_single_rows, ctx.seg_start,
                           ctx.positions, table, scale, window, ctx.max_context)
    # the one launch
    one = torch.full((R, H * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    part_o.fill_(float("nan"))
    part_ml.fill_(float("nan"))
    ops().attention_decode_qkv(qkv.to(DEV), qw_d, kw_d, 1e-5, inv_d, k_cache, v_cache, one, part_o, part_ml,
                               ctx.single_rows, ctx.n_single_rows, ctx.seg_start, ctx.positions, table, H, scale,
                               window, ctx.max_context, interleaved=interleaved)
    one_f, two_f = one.cpu().float().reshape(R, H, D), two.cpu().float().reshape(R, H, D)
    torch.testing.assert_close(one_f, ref, rtol=2 ** -6, atol=2 ** -6)
    torch.testing.assert_close(one_f, two_f, rtol=2 ** -6, atol=2 ** -6)
    # the new keys and values are in their pages, as the other launch leaves them up to one rounding, and nothing else is
    for r, c in enumerate(ctx_lens):
        page, slot = tables[r][(c - 1) // page_size], (c - 1) % page_size
        torch.testing.assert_close(k_cache[page, :, slot].cpu().float(), new_k[r], rtol=2 ** -7, atol=2 ** -7)
        assert torch.equal(v_cache[page, :, :, slot].cpu().float(), new_v[r])
    assert torch.equal(torch.isnan(k_cache), torch.isnan(k2)) and torch.equal(torch.isnan(v_cache), torch.isnan(v2))
    assert int((~torch.isnan(k_cache[:, 0, :, 0])).sum()) == sum(ctx_lens)


def test_matrix_core_attention_refuses_other_sizes():
    from imparo_amd.kernels import KernelArgumentError
    assert not ops().mfma_attention_supported(torch.bfloat16, 8, 64)
    assert not ops().mfma_attention_supported(torch.float32, 16, 64)
    assert not ops().mfma_attention_supported(torch.bfloat16, 16, 144)
    assert ops().mfma_attention_supported(torch.bfloat16, 64, 112)
    q = torch.zeros(1, 2, 144, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(2, 1, 16, 144, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(2, 1, 144, 16, dtype=torch.bfloat16, device=DEV)
    i = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelArgumentError, match="head sizes"):
        ops().attention_prefill(q, kc, vc, torch.zeros(1, 288, dtype=torch.bfloat16, device=DEV), i, 1, 1, i, i, i,
                                torch.zeros(1, 1, dtype=torch.int32, device=DEV), 1.0, None)


@pytest.mark.parametrize("kernel", ["wave", "mfma"])
@pytest.mark.parametrize("where", ["first", "page_edge", "middle"])
def test_attention_finds_one_far_key_among_hundreds(where, kernel):
    pick = {"first": lambda c: 0, "page_edge": lambda c: (c // 2 // 16) * 16, "middle": lambda c: c // 3}[where]
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2 ** -6)):
        if kernel == "mfma" and dtype == torch.float32:
            continue
        got, ref = _attention_case(4, 2, 64, 16, None, dtype, sharpen=pick, kernel=kernel)
        torch.testing.assert_close(got, ref, rtol=tol, atol=tol)
        # the test means something: with the far key the last query's output is that key's value
    # the last row's query sits at 199 and its far key at 66: a window of 133 starts at 67 and
    # leaves it out, one of 134 starts at 66 and takes it in; the edge decides the output
    for window, dtype in ((133, torch.float32), (134, torch.float32), (133, torch.bfloat16), (134, torch.bfloat16)):
        if kernel == "mfma" and dtype == torch.float32:
            continue
        got, ref = _attention_case(2, 1, 32, 16 if kernel == "mfma" else 8, window, dtype, sharpen=lambda c: c // 3,
                                   kernel=kernel)
        torch.testing.assert_close(got, ref, rtol=2 ** -6, atol=2 ** -6)


# ---------------------------------------------------------------- short conv
@pytest.mark.parametrize("width,taps", [(8, 2), (100, 3), (300, 4), (64, 7)])
def test_short_conv(width, taps):
    segments = [(0, 1), (0, 9), (0, 2), (0, 40)]            # segments shorter than the history too
    slots = [3, 0, 5, 1]
    w = rnd(width, 1, taps, seed=1, scale=0.3)
    bias = rnd(width, seed=2, scale=0.1)
    for use_bias in (False, True):
        ctx = hand_context(segments, 16, 16, torch.float32, DEV, fixed_sites={0: (taps - 1, width)}, slots=slots)
        state = ctx.fixed_state(0)
        state0 = rnd(8, taps - 1, width, seed=3)
        state.copy_(state0)
        bcx = rnd(ctx.n_tokens, 3 * width, seed=4)
        for out_dtype in (torch.float32, torch.bfloat16):
            state.copy_(state0)
            out = torch.empty(ctx.n_tokens, width, dtype=out_dtype, device=DEV)
            ops().short_conv(bcx.to(DEV), w.reshape(width, taps).to(DEV), bias.to(DEV) if use_bias else None, state,
                             ctx.row_of_token, ctx.seg_start, ctx.seg_len, ctx.slot, out)
            at = 0
            for (p0, n), slot in zip(segments, slots):
                y, s = P.short_conv(bcx[at:at + n], w, bias if use_bias else None, state=state0[slot])
                tol = dict(rtol=1e-5, atol=1e-5) if out_dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
                torch.testing.assert_close(out[at:at + n].cpu().float(), y, **tol)
                torch.testing.assert_close(state[slot].cpu(), s, rtol=1e-6, atol=1e-6)
                at += n
            for slot in set(range(8)) - set(slots):          # other requests' state is left alone
                assert torch.equal(state[slot].cpu(), state0[slot])


@pytest.mark.parametrize("width,taps", [(8, 2), (100, 3), (300, 4), (64, 7)])
def test_short_conv_single_tokens_in_one_launch(width, taps):
    """The fused kernel for batches of single tokens gives the same bits as the general pair."""
    segments = [(5, 1), (0, 1), (9, 1)]
    slots = [4, 1, 6]
    w = rnd(width, taps, seed=1, scale=0.3).to(DEV)
    bias = rnd(width, seed=2, scale=0.1).to(DEV)
    bcx = rnd(3, 3 * width, seed=4).to(DEV)
    state0 = rnd(8, taps - 1, width, seed=3)
    results = []
    for single in (False, True):
        ctx = hand_context(segments, 16, 16, torch.float32, DEV, fixed_sites={0: (taps - 1, width)}, slots=slots)
        state = ctx.fixed_state(0)
        state.copy_(state0)
        out = torch.empty(3, width, device=DEV)
        ops().short_conv(bcx, w, bias, state, ctx.row_of_token, ctx.seg_start, ctx.seg_len, ctx.slot, out,
                         single_tokens=single)
        results.append((out.cpu(), state.cpu().clone()))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])
    y, s = P.short_conv(bcx[1:2].cpu(), w.cpu().reshape(width, 1, taps), bias.cpu(), state=state0[1])
    torch.testing.assert_close(results[1][0][1:2], y, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(results[1][1][1], s, rtol=1e-6, atol=1e-6)


def test_short_conv_exact_vectors_from_the_reference():
    # /root/reference/crates/imparo-cpu/src/ops.rs:1207-1254 on the GPU kernel
    ctx = hand_context([(0, 2)], 16, 4, torch.float32, DEV, fixed_sites={0: (2, 1)})
    state = ctx.fixed_state(0)
    state[0] = torch.tensor([[5.0], [7.0]])
    out = torch.empty(2, 1, device=DEV)
    ops().short_conv(torch.ones(2, 3, device=DEV), torch.tensor([[1.0, 0.0, 0.0]], device=DEV), None, state,
                     ctx.row_of_token, ctx.seg_start, ctx.seg_len, ctx.slot, out)
    assert out.flatten().tolist() == [5.0, 7.0] and state[0].flatten().tolist() == [1.0, 1.0]


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("width,k,taps", [(16, 264, 2), (200, 1024, 3), (64, 2048, 4), (40, 512, 6), (24, 4608, 3)])
def test_in_proj_and_conv_in_one_launch(m, width, k, taps):
    """A decode step's rows: the projection to [B | C | x] and the gated conv in one launch give what
    the two launches give (the same bits where both split K over the same waves), and shift the state."""
    x = rnd(m, k, seed=1).to(torch.bfloat16).to(DEV)
    w_in = rnd(3 * width, k, seed=2, scale=0.05).to(torch.bfloat16).to(DEV)
    b_in = rnd(3 * width, seed=3, scale=0.1).to(DEV)
    w = rnd(width, taps, seed=4, scale=0.3).to(DEV)
    b = rnd(width, seed=5, scale=0.1).to(DEV)
    state0 = rnd(20, taps - 1, width, seed=6)
    slots = torch.randperm(20, generator=torch.Generator().manual_seed(7))[:m].to(torch.int32)
    for use_bias in (True, False):
        for out_dtype in (torch.float32, torch.bfloat16):
            ctx = hand_context([(3, 1)] * m, 16, 2 * m, torch.float32, DEV, fixed_sites={0: (taps - 1, width)},
                               n_slots=20, slots=slots.tolist())
            state = ctx.fixed_state(0)
            state.copy_(state0)
            bcx = torch.empty(m, 3 * width, device=DEV)
            ops().gemm(x, w_in, bcx, bias=b_in if use_bias else None)
            two = torch.empty(m, width, dtype=out_dtype, device=DEV)
            ops().short_conv(bcx, w, b if use_bias else None, state, ctx.row_of_token, ctx.seg_start, ctx.seg_len,
                             ctx.slot, two, single_tokens=True)
            state_two = state.cpu().clone()
            state.copy_(state0)
            one = torch.full((m, width), float("nan"), dtype=out_dtype, device=DEV)
            ops().in_proj_conv_decode(x, w_in, b_in if use_bias else None, w, b if use_bias else None, state,
                                      ctx.slot, one)
            if k <= 2048:
                assert torch.equal(one.cpu(), two.cpu()) and torch.equal(state.cpu(), state_two)
            else:
                tol = dict(rtol=1e-5, atol=1e-5) if out_dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
                torch.testing.assert_close(one.cpu().float(), two.cpu().float(), **tol)
                torch.testing.assert_close(state.cpu(), state_two, rtol=1e-5, atol=1e-5)
            untouched = [s for s in range(20) if s not in slots.tolist()]
            assert torch.equal(state.cpu()[untouched], state0[untouched])
    from imparo_amd.kernels import KernelArgumentError
    with pytest.raises(KernelArgumentError, match="16"):
        ops().in_proj_conv_decode(torch.zeros(17, k, dtype=torch.bfloat16, device=DEV), w_in, None, w, None, state,
                                  torch.zeros(17, dtype=torch.int32, device=DEV), torch.empty(17, width, device=DEV))


# ---------------------------------------------------------------- sampling
@pytest.mark.parametrize("vocab", [7, 200, 1000, 65536, 70001])
def test_argmax_rows(vocab):
    x = rnd(6, vocab, seed=vocab)
    x[1, vocab // 2] = x[1].max() + 1
    x[1, vocab - 1] = x[1, vocab // 2]               # a tie: the smaller index wins
    x[2, 0] = float("nan")
    x[3] = float("nan")                               # all NaN -> 0
    x[4, :] = -float("inf")
    x[5, vocab - 1] = 50.0
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    ops().argmax_rows(x.to(DEV), out)
    assert out.cpu().tolist() == [P.argmax_first(r.numpy()) for r in x]
    assert out[1].item() == vocab // 2 and out[3].item() == 0 and out[5].item() == vocab - 1


@pytest.mark.parametrize("vocab", [7, 384, 65536])
def test_sample_rows(vocab):
    n = 64
    logits = rnd(n, vocab, seed=1, scale=2.0)
    temps = torch.tensor([0.8] * (n - 2) + [0.0, 1.7])
    g = torch.Generator().manual_seed(2)
    u = torch.rand(n, generator=g)
    u[0], u[1] = 0.0, 0.99999994
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample_rows(logits.to(DEV), temps.to(DEV), u.to(DEV), out)
    got = out.cpu().tolist()
    for r in range(n):
        if temps[r] <= 0:
            assert got[r] == P.argmax_first(logits[r].numpy())
            continue
        p = torch.softmax(logits[r].double() / temps[r].double(), dim=0)
        cdf = torch.cumsum(p, 0)
        target = float(u[r])
        lo = float(cdf[got[r] - 1]) if got[r] > 0 else 0.0
        hi = float(cdf[got[r]])
        # the pick's interval of the CDF holds the target, up to float32 rounding of the sums
        assert lo - 1e-5 <= target <= hi + 1e-5, (r, got[r], lo, target, hi)
    # draws follow the distribution: a row repeated with many uniforms
    row = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]]).repeat(4000, 1)
    uu = torch.rand(4000, generator=g)
    out = torch.empty(4000, dtype=torch.int32, device=DEV)
    ops().sample_rows(row.to(DEV), torch.full((4000,), 1.0, device=DEV), uu.to(DEV), out)
    freq = torch.bincount(out.cpu().long(), minlength=5).float() / 4000
    assert (freq - torch.softmax(row[0], 0)).abs().max() < 0.03


# ---------------------------------------------------------------- products with a folded norm (at most 16 rows)
from imparo_amd.kernels import ops as _rows_ops
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (5, 200, 136), (13, 1536, 1536), (16, 2048, 8192), (8, 96, 320),
                                   (16, 4608, 1024), (3, 13824, 1536)])
def test_rows_product_added_to_the_stream_leaves_sums_of_squares_and_weighted_rows(m, n, k):
    dev = "cuda:0"
    g = torch.Generator().manual_seed(m * 1000 + n + k)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    bias = torch.randn(n, generator=g) * 0.1
    stream = torch.randn(m, n, generator=g)
    by = 1.0 + 0.1 * torch.randn(n, generator=g)
    want = stream + x.float() @ w.float().t() + bias
    into = stream.clone().to(dev)
    parts = _rows_ops.rows_parts(n)
    ssq = torch.full((parts, 16), 7.0, device=dev)
    weighted = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    _rows_ops.rows_gemm(x.to(dev), w.to(dev), bias=bias.to(dev), into=into, ssq_out=ssq, weighted_out=weighted,
                  weighted_by=by.to(dev))
    torch.testing.assert_close(into.cpu(), want, rtol=2e-5, atol=2e-5 * float(want.abs().max()))
    got_ssq = ssq.cpu().sum(0)
    torch.testing.assert_close(got_ssq[:m], (into.cpu() ** 2).sum(-1), rtol=1e-5, atol=0)
    assert float(got_ssq[m:].abs().max()) == 0.0 if m < 16 else True      # rows the step does not have: zero
    torch.testing.assert_close(weighted.cpu().float(), (into.cpu() * by).to(torch.bfloat16).float(), rtol=2 ** -7, atol=1e-6)


@pytest.mark.parametrize("swiglu", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (5, 200, 136), (13, 4608, 1536), (16, 16384, 2048), (9, 96, 320),
                                   (16, 9216, 1024), (2, 3072, 2048)])
def test_rows_product_scales_its_rows_at_the_end(m, n, k, swiglu):
    """The activations are the stream times a norm's weight, rounded to bfloat16; the sums of squares come
    in parts; the product must equal (rows * rsqrt(mean square + eps)) . W^T in float32."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(m + n + k)
    stream = torch.randn(m, k, generator=g) * 3.0
    norm_w = 1.0 + 0.1 * torch.randn(k, generator=g)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    eps = 1e-5
    weighted = (stream * norm_w).to(torch.bfloat16)
    n_parts = 37
    cut = torch.linspace(0, k, n_parts + 1).long()
    ssq = torch.zeros(n_parts, 16)
    for p in range(n_parts):
        ssq[p, :m] = (stream[:, cut[p]:cut[p + 1]] ** 2).sum(-1)
    scale = torch.rsqrt((stream ** 2).mean(-1, keepdim=True) + eps)
    want = (weighted.float() @ w.float().t()) * scale
    if swiglu:
        want = torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2]
    for out_dtype in (torch.float32, torch.bfloat16):
        out = torch.zeros(m, n // 2 if swiglu else n, dtype=out_dtype, device=dev)
        _rows_ops.rows_gemm(weighted.to(dev), w.to(dev), out=out, swiglu=swiglu, ssq_in=ssq.to(dev), eps=eps)
        tol = 2e-5 if out_dtype == torch.float32 else 2 ** -7
        torch.testing.assert_close(out.cpu().float(), want, rtol=tol, atol=tol * float(want.abs().max()))
