"""The decode attention entry point that allocates nothing
(imparo_attention_decode_static): called through ctypes, held bit for bit
against imparo_attention_decode with a workspace, on two calls in a row, the
second with a smaller input, so that what the first call left in the library's
own buffer must not show."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
SPLIT = 256
SCRATCH_BYTES = 16 << 20
TOO_SMALL = 3


def _lib():
    from imparo_amd.kernels.library import loaded_path
    lib = ctypes.CDLL(loaded_path())
    lib.imparo_attention_decode.argtypes = [P, P, P, P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P]
    lib.imparo_attention_decode.restype = I
    lib.imparo_attention_decode_static.argtypes = [P, P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P]
    lib.imparo_attention_decode_static.restype = I
    return lib


def _case(contexts, heads, kv_heads, head_dim, page_size, seed):
    """Single-token rows with the given context lengths over a shuffled paged cache."""
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(seed)
    n = len(contexts)
    width = max(-(-c // page_size) for c in contexts)
    n_pages = n * width + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((n, width), -1, dtype=torch.int32)
    for r, c in enumerate(contexts):
        for j in range(-(-c // page_size)):
            table[r, j] = order.pop()
    k = torch.randn(n_pages, kv_heads, page_size, head_dim, generator=g).to(torch.bfloat16)
    v = torch.randn(n_pages, kv_heads, head_dim, page_size, generator=g).to(torch.bfloat16)
    q = torch.randn(n, heads, head_dim, generator=g).to(torch.bfloat16)
    t = dict(q=q, k=k, v=v, table=table,
             rows=torch.arange(n, dtype=torch.int32), seg_start=torch.arange(n, dtype=torch.int32),
             positions=torch.tensor([c - 1 for c in contexts], dtype=torch.int32))
    t = {name: x.to(dev).contiguous() for name, x in t.items()}
    t.update(n=n, heads=heads, kv_heads=kv_heads, head_dim=head_dim, page_size=page_size, n_pages=n_pages,
             width=width, n_splits=-(-max(contexts) // SPLIT), scale=1.0 / math.sqrt(head_dim))
    return t


def _run(lib, t, static: bool) -> torch.Tensor:
    dev = t["q"].device
    out = torch.full((t["n"], t["heads"] * t["head_dim"]), float("nan"), dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    tail = (t["rows"].data_ptr(), t["n"], t["seg_start"].data_ptr(), t["positions"].data_ptr(),
            t["table"].data_ptr(), t["width"], t["page_size"], t["heads"], t["kv_heads"], t["head_dim"],
            t["n_pages"], t["scale"], 0, t["n_splits"], stream)
    head = (t["q"].data_ptr(), t["k"].data_ptr(), t["v"].data_ptr(), out.data_ptr())
    if static:
        status = lib.imparo_attention_decode_static(*head, *tail)
    else:
        slots = t["n"] * t["heads"] * t["n_splits"]
        part_o = torch.full((slots * t["head_dim"],), float("nan"), device=dev)
        part_ml = torch.full((slots * 2,), float("nan"), device=dev)
        status = lib.imparo_attention_decode(*head, part_o.data_ptr(), part_ml.data_ptr(), *tail)
    assert status == 0, f"status {status}"
    torch.cuda.synchronize()
    return out.float().cpu()


def test_static_scratch_decode_equals_the_workspace_one_twice_in_a_row():
    lib = _lib()
    big = _case([1500, 700, 257, 2048, 33, 1024], heads=8, kv_heads=2, head_dim=64, page_size=64, seed=11)
    small = _case([300, 5], heads=8, kv_heads=2, head_dim=64, page_size=64, seed=12)
    want_big, want_small = _run(lib, big, static=False), _run(lib, small, static=False)
    assert torch.isfinite(want_big).all() and torch.isfinite(want_small).all()
    before = torch.cuda.memory_allocated()
    got_big = _run(lib, big, static=True)
    got_small = _run(lib, small, static=True)     # the buffer still holds the first call's partial results
    assert torch.equal(got_big, want_big)
    assert torch.equal(got_small, want_small)
    assert torch.cuda.memory_allocated() == before
    # and once more in the other order, in the same process
    assert torch.equal(_run(lib, small, static=True), want_small)
    assert torch.equal(_run(lib, big, static=True), want_big)


def test_static_scratch_decode_refuses_what_does_not_fit():
    lib = _lib()
    t = _case([64, 64], heads=8, kv_heads=2, head_dim=64, page_size=64, seed=13)
    # as many splits as would need more than the library's buffer; the refusal comes before any launch
    slots_that_fit = SCRATCH_BYTES // 4 // (t["head_dim"] + 2)
    t["n_splits"] = slots_that_fit // (t["n"] * t["heads"]) + 64
    dev = t["q"].device
    out = torch.zeros((t["n"], t["heads"] * t["head_dim"]), dtype=torch.bfloat16, device=dev)
    status = lib.imparo_attention_decode_static(
        t["q"].data_ptr(), t["k"].data_ptr(), t["v"].data_ptr(), out.data_ptr(), t["rows"].data_ptr(), t["n"],
        t["seg_start"].data_ptr(), t["positions"].data_ptr(), t["table"].data_ptr(), t["width"], t["page_size"],
        t["heads"], t["kv_heads"], t["head_dim"], t["n_pages"], t["scale"], 0, t["n_splits"],
        torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert status == TOO_SMALL
    assert not out.any()
