"""Each part alone, built from its spec and a handful of tensors, stepped on a
hand-made batch and compared with the plain functions."""
import math

import pytest
import torch

import plain_lfm2 as P
from gpu_helpers import hand_context

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part_adds_the_pending_delta(dtype):
    from imparo_amd.config import PartSpec
    from imparo_amd.parts import part_class, Residual
    spec = PartSpec("rms_norm", "n", dict(width=72, eps=1e-3))
    w = 1 + 0.1 * rnd(72, seed=1)
    norm = part_class("norm", "rms_norm")(spec, {"n.weight": w.to(torch.bfloat16)}, DEV, dtype)
    ctx = hand_context([(0, 6)], 16, 4, dtype, DEV)
    x, d = rnd(6, 72, seed=2), rnd(6, 72, seed=3)
    res = Residual(x.to(DEV).clone(), d.to(DEV))
    h = norm.forward(ctx, res, dtype)
    assert res.pending is None and torch.equal(res.x.cpu(), x + d)
    torch.testing.assert_close(h.cpu().float(), P.rms_norm(x + d, w.to(torch.bfloat16).float(), 1e-3), **tol(dtype))
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    res = Residual(x.to(DEV).clone(), d.to(DEV))
    h = norm.forward_rows(ctx, res, rows, torch.float32)
    torch.testing.assert_close(h.cpu(), P.rms_norm((x + d)[[4, 1]], w.to(torch.bfloat16).float(), 1e-3), rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,Hk,D,window,rot", [(6, 2, 32, None, 32), (4, 4, 16, 11, 8), (3, 1, 64, None, 0)])
def test_attention_part(dtype, H, Hk, D, window, rot):
    """Two requests in two steps each (a portion, then the rest beside a
    decode token of the other): the part fills its own cache as it goes."""
    from imparo_amd.config import PartSpec
    from imparo_amd.parts import part_class
    E = 40
    spec = PartSpec("attention", "a", dict(
        width=E, heads=H, kv_heads=Hk, head_dim=D, scale=1.0 / math.sqrt(D), window=window,
        qk_norm=PartSpec("rms_norm", "", dict(width=D, eps=1e-5)),
        position=PartSpec("rope_neox", "", dict(base=500.0, rotary_dim=rot)) if rot else PartSpec("none")))
    cls = part_class("mixer", "attention")
    t = {}
    for i, (name, (decl, init)) in enumerate(sorted(cls.declare(spec).items())):
        v = (1 + 0.1 * rnd(*decl.shape, seed=i)) if init == "norm" else rnd(*decl.shape, seed=i, scale=0.15)
        t[name] = v.to(torch.bfloat16)
    part = cls(spec, t, DEV, dtype)
    # the part says how its cache is laid out (V transposed in a page where its matrix-core kernels apply)
    from imparo_amd.cache import kv_spec
    vt = dtype == torch.bfloat16
    assert part.cache_spec(16) == kv_spec(Hk, D, window, v_transposed=vt) and part.v_transposed == vt
    f = {k: v.float() for k, v in t.items()}
    lens = [23, 14]
    hs = [rnd(n, E, seed=50 + r).to(torch.bfloat16).float() for r, n in enumerate(lens)]
    refs = []
    for h in hs:
        T = h.shape[0]
        pos = list(range(T))
        q = P.rms_norm(P.linear(h, f["a.q_proj.weight"]).reshape(T, H, D), f["a.q_norm.weight"], 1e-5)
        k = P.rms_norm(P.linear(h, f["a.k_proj.weight"]).reshape(T, Hk, D), f["a.k_norm.weight"], 1e-5)
        v = P.linear(h, f["a.v_proj.weight"]).reshape(T, Hk, D)
        if rot:
            q, k = P.rope_neox(q, pos, 500.0, rot), P.rope_neox(k, pos, 500.0, rot)
        o = P.attend(q, k, v, pos, 1.0 / math.sqrt(D), window)
        refs.append(P.linear(o.reshape(T, H * D), f["a.o_proj.weight"]))
    tables = [[5, 2], [0]]
    ctx1 = hand_context([(0, 20), (0, 13)], 16, 8, dtype, DEV, kv_sites={3: (Hk, D)}, tables=tables, v_transposed=vt)
    x1 = torch.cat([hs[0][:20], hs[1][:13]]).to(part.in_dtype).to(DEV)
    out1 = part.forward(ctx1, 3, True, x1).cpu().clone()
    ctx2 = hand_context([(20, 3), (13, 1)], 16, 8, dtype, DEV, kv_sites={3: (Hk, D)}, tables=tables, v_transposed=vt)
    ctx2.storage = ctx1.storage
    x2 = torch.cat([hs[0][20:], hs[1][13:]]).to(part.in_dtype).to(DEV)
    out2 = part.forward(ctx2, 3, True, x2).cpu()
    got0 = torch.cat([out1[:20], out2[:3]])
    got1 = torch.cat([out1[20:], out2[3:]])
    torch.testing.assert_close(got0, refs[0], **tol(dtype))
    torch.testing.assert_close(got1, refs[1], **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,bias", [(3, False), (4, True), (2, True)])
def test_short_conv_part(dtype, taps, bias):
    from imparo_amd.config import PartSpec
    from imparo_amd.parts import part_class
    from imparo_amd.cache import FixedSpec
    E = 56
    spec = PartSpec("short_conv", "c", dict(width=E, taps=taps, bias=bias))
    cls = part_class("mixer", "short_conv")
    t = {}
    for i, (name, (decl, init)) in enumerate(sorted(cls.declare(spec).items())):
        t[name] = rnd(*decl.shape, seed=i, scale=0.3 if init == "conv" else 0.15).to(torch.bfloat16)
    part = cls(spec, t, DEV, dtype)
    assert part.cache_spec(16) == FixedSpec((taps - 1, E))
    f = {k: v.float() for k, v in t.items()}
    b = (lambda n: f[f"c.{n}.bias"]) if bias else (lambda n: None)
    h = rnd(17, E, seed=9).to(torch.bfloat16).float()
    bcx = P.linear(h, f["c.in_proj.weight"], b("in_proj"))
    y, _ = P.short_conv(bcx, f["c.conv.weight"], b("conv"))
    ref = P.linear(y, f["c.out_proj.weight"], b("out_proj"))
    # 17 tokens as 1 + 9 + 2 + 5, the state carried in slot 2 of site 7
    outs, at = [], 0
    storage = None
    for n in (1, 9, 2, 5):
        ctx = hand_context([(at, n)], 16, 4, dtype, DEV, fixed_sites={7: (taps - 1, E)}, slots=[2])
        if storage is not None:
            ctx.storage = storage
        storage = ctx.storage
        outs.append(part.forward(ctx, 7, True, h[at:at + n].to(part.in_dtype).to(DEV)).cpu().clone())
        at += n
    torch.testing.assert_close(torch.cat(outs), ref, **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_embedding_and_head_parts(dtype):
    from imparo_amd.config import PartSpec
    from imparo_amd.parts import part_class
    E, F, V = 48, 104, 77
    ffn_spec = PartSpec("swiglu", "f", dict(width=E, hidden=F, names=dict(gate="w1", up="w3", down="w2")))
    t = {"f.w1.weight": rnd(F, E, seed=1, scale=0.2), "f.w3.weight": rnd(F, E, seed=2, scale=0.2),
         "f.w2.weight": rnd(E, F, seed=3, scale=0.2), "e.weight": rnd(V, E, seed=4)}
    t = {k: v.to(torch.bfloat16) for k, v in t.items()}
    f = {k: v.float() for k, v in t.items()}
    ctx = hand_context([(0, 70)], 16, 8, dtype, DEV)      # 70 rows: the many-rows GEMM; 9 rows: the few-rows one
    ffn = part_class("feed_forward", "swiglu")(ffn_spec, t, DEV, dtype)
    for n in (70, 9):
        x = rnd(n, E, seed=5).to(torch.bfloat16).float()
        got = ffn.forward(ctx, x.to(ffn.in_dtype).to(DEV)).cpu()
        torch.testing.assert_close(got, P.swiglu(x, f["f.w1.weight"], f["f.w3.weight"], f["f.w2.weight"]), **tol(dtype))
    placed = {}
    emb = part_class("embedding", "embedding")(PartSpec("embedding", "e", dict(vocab=V, width=E)), t, DEV, dtype, placed)
    head = part_class("head", "linear_head")(PartSpec("linear_head", "e", dict(vocab=V, width=E)), t, DEV, dtype, placed)
    assert head.proj.weight.data_ptr() == emb.table.data_ptr()         # tied: one tensor on the device
    ids = torch.tensor([76, 0, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(ctx, ids).cpu(), f["e.weight"][[76, 0, 3]])
    x = rnd(3, E, seed=6).to(torch.bfloat16).float()
    torch.testing.assert_close(head.forward(ctx, x.to(head.in_dtype).to(DEV)).cpu(), P.linear(x, f["e.weight"]), **tol(dtype))


def test_a_matrix_stored_in_float32_runs_in_float32_under_a_bfloat16_engine():
    from imparo_amd.parts import Linear, place_matrix
    w32 = rnd(24, 40, seed=1)
    lin = Linear(place_matrix(w32, torch.bfloat16, DEV))
    assert lin.in_dtype == torch.float32
    lin16 = Linear(place_matrix(w32.to(torch.bfloat16), torch.bfloat16, DEV))
    assert lin16.in_dtype == torch.bfloat16
    assert Linear(place_matrix(w32.to(torch.bfloat16), torch.float32, DEV)).in_dtype == torch.float32
