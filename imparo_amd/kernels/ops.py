"""Python faces of the gfx950 kernels.

Each function checks on the host what its kernel assumes (device, dtype,
contiguity, shapes, index ranges that the host knows), then launches on the
current stream. There is no CPU path: a tensor that is not on the GPU is an
error, and so is a missing kernel library.
"""
from __future__ import annotations

from typing import Optional

import torch

from .library import library

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def _code(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _CODES:
        raise KernelArgumentError(f"{what} has dtype {t.dtype}; kernels take float32 or bfloat16")
    return _CODES[t.dtype]


def _dev(t: Optional[torch.Tensor], what: str, dtype=None, shape=None) -> int:
    """Checks a tensor and returns its device address (0 for None)."""
    if t is None:
        return 0
    if not isinstance(t, torch.Tensor):
        raise KernelArgumentError(f"{what} is not a tensor")
    if t.device.type != "cuda":
        raise KernelArgumentError(f"{what} is on {t.device}; the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelArgumentError(f"{what} is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelArgumentError(f"{what} has dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelArgumentError(f"{what} has shape {list(t.shape)}, expected {list(shape)}")
    return t.data_ptr()


_launch_stream: Optional[int] = None


class on_current_stream:
    """For a run of launches that all go to the stream that is current now (a
    step's hundred kernels, also under graph capture): looks the stream up once
    instead of once per launch, which costs more host time than the launch."""

    def __enter__(self):
        global _launch_stream
        self._before = _launch_stream
        _launch_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _launch_stream
        _launch_stream = self._before
        return False


def _stream() -> int:
    if _launch_stream is not None:
        return _launch_stream
    return torch.cuda.current_stream().cuda_stream


def _check(status: int, name: str) -> None:
    if status == 0:
        return
    why = {1: "an argument was refused (size or pointer the kernel cannot take)",
           2: "the launch failed"}.get(status, f"status {status}")
    raise KernelArgumentError(f"{name}: {why}")


def load_code() -> None:
    """Loads every kernel file's code onto the current device (the runtime would do so at each
    file's first launch, which a stream under graph capture cannot)."""
    _check(library().imparo_load_code(), "load_code")


def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    vocab, width = table.shape
    n = ids.shape[0]
    _check(library().imparo_embed_gather(
        _dev(table, "embedding table"), _code(table, "embedding table"),
        _dev(ids, "token ids", torch.int32, (n,)), _dev(out, "embedding output", torch.float32, (n, width)),
        n, width, vocab, _stream()), "embed_gather")
    return out


def place_tokens(ids: torch.Tensor, dst: torch.Tensor, src: torch.Tensor, src_index: torch.Tensor,
                 vocab: int) -> torch.Tensor:
    """ids[dst[i]] = src[src_index[i]]: token ids that the step before sampled and that were
    not read back. The caller has checked the indices on the host (they come from there)."""
    n = dst.shape[0]
    _check(library().imparo_place_tokens(
        _dev(ids, "token ids", torch.int32), _dev(dst, "places", torch.int32, (n,)),
        _dev(src, "sampled tokens", torch.int32), _dev(src_index, "indices of sampled tokens", torch.int32, (n,)),
        n, vocab, _stream()), "place_tokens")
    return ids


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             write_back: bool = False) -> torch.Tensor:
    """out[i] = norm(x[src] (+ delta[src])) * weight, src = rows[i] or i.
    `delta` is shaped like x, or [slices, *x.shape]: slices are added in order.
    write_back stores x + delta into x (only without rows)."""
    width = x.shape[-1]
    n_out = out.shape[0]
    if rows is None and n_out != x.shape[0]:
        raise KernelArgumentError(f"rms_norm: out has {n_out} rows, x has {x.shape[0]}")
    if rows is not None and rows.shape[0] != n_out:
        raise KernelArgumentError("rms_norm: one source row index per output row is needed")
    if write_back and (rows is not None or delta is None):
        raise KernelArgumentError("rms_norm: write_back needs a delta and no row selection")
    n_delta = 0
    if delta is not None:
        n_delta = delta.shape[0] if delta.dim() == x.dim() + 1 else 1
        want = (n_delta,) + tuple(x.shape) if delta.dim() == x.dim() + 1 else tuple(x.shape)
        _dev(delta, "rms_norm delta", torch.float32, want)
    _check(library().imparo_rms_norm(
        _dev(x, "rms_norm x", torch.float32), _dev(delta, "rms_norm delta", torch.float32), n_delta, x.shape[0],
        _dev(rows, "rms_norm rows", torch.int32), _dev(weight, "rms_norm weight", torch.float32, (width,)),
        _dev(out, "rms_norm out", None, (n_out, width)), _code(out, "rms_norm out"),
        n_out, width, float(eps), int(write_back), _stream()), "rms_norm")
    return out


def gemm_slices(m: int, n: int, k: int, dtype: torch.dtype) -> int:
    """Into how many slices of K this product may be cut when its consumer adds the slices (1: none)."""
    return int(library().imparo_gemm_slices(m, n, k, _CODES.get(dtype, -1)))


def gemm_adds(m: int, n: int, k: int, dtype: torch.dtype) -> bool:
    """Whether `gemm(..., add=True)` is taken for this shape (many rows on the tile kernel, K in one piece)."""
    return bool(library().imparo_gemm_adds(m, n, k, _CODES.get(dtype, -1)))


def gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
         swiglu: bool = False, variant: int = 0, add: bool = False) -> torch.Tensor:
    """out[m, n] = x[m, k] . w[n, k]^T (+ bias[n]); x and w share a dtype; float32
    accumulate. With `swiglu` the rows of w alternate gate and up and out is
    [m, n/2] = silu(gate) * up. An `out` of shape [slices, m, n] (slices =
    gemm_slices(...)) receives the sums over slices of K, to be added by the consumer.
    With `add` (float32 out, where gemm_adds(...) says so) the product is added to what `out` holds.
    `variant` other than 0 names the kernel (tests and measurements only; see imparo_gemm_variant)."""
    m, k = x.shape
    n, kw = w.shape
    if kw != k:
        raise KernelArgumentError(f"gemm: x has {k} columns but the weight has {kw}")
    if x.dtype != w.dtype:
        raise KernelArgumentError(f"gemm: x is {x.dtype} but the weight is {w.dtype}")
    if x.dtype == torch.bfloat16 and k % 8 != 0:
        raise KernelArgumentError(f"gemm: the bfloat16 kernels need the inner size to be a multiple of 8, got {k}")
    if swiglu and n % 2:
        raise KernelArgumentError("gemm: a gate/up weight has an even number of rows")
    slices = 1
    if out.dim() == 3:
        slices = out.shape[0]
        if (slices != gemm_slices(m, n, k, x.dtype) and not variant) or swiglu or out.dtype != torch.float32:
            raise KernelArgumentError(f"gemm: this product cannot be cut into {slices} slices of K")
        _dev(out, "gemm out", torch.float32, (slices, m, n))
    else:
        _dev(out, "gemm out", None, (m, n // 2 if swiglu else n))
    if add and (swiglu or slices != 1 or variant or out.dtype != torch.float32 or not gemm_adds(m, n, k, x.dtype)):
        raise KernelArgumentError("gemm: this product cannot be added to what its output holds")
    args = (_dev(x, "gemm x"), _dev(w, "gemm weight"), _dev(bias, "gemm bias", torch.float32, (n,)),
            out.data_ptr(), _code(x, "gemm x"), _code(out, "gemm out"), m, n, k, 2 if add else int(swiglu), slices)
    if variant:
        _check(library().imparo_gemm_variant(*args, int(variant), _stream()), "gemm")
    else:
        _check(library().imparo_gemm(*args, _stream()), "gemm")
    return out


def qk_norm_rope_store(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                       eps: float, inv_freq: Optional[torch.Tensor], positions: torch.Tensor,
                       row_of_token: torch.Tensor, block_table: Optional[torch.Tensor], page_size: int,
                       q_out: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                       heads: int, kv_heads: int, head_dim: int, v_transposed: bool = False,
                       interleaved: bool = False) -> torch.Tensor:
    """`inv_freq` [n] turns pair i by position * inv_freq[i]: pair i is dims (i, i + n), or with
    `interleaved` dims (2i, 2i + 1)."""
    n = qkv.shape[0]
    units = heads + 2 * kv_heads
    write_kv = k_cache is not None
    n_freq = 0 if inv_freq is None else inv_freq.shape[0]
    n_pages = 0
    table_stride = 0
    if write_kv:
        n_pages = k_cache.shape[0]
        _dev(k_cache, "k cache", q_out.dtype, (n_pages, kv_heads, page_size, head_dim))
        _dev(v_cache, "v cache", q_out.dtype, (n_pages, kv_heads, head_dim, page_size) if v_transposed
             else (n_pages, kv_heads, page_size, head_dim))
        if block_table is None or block_table.dim() != 2:
            raise KernelArgumentError("qk_norm_rope_store: a [rows, pages] block table is needed to write the cache")
        table_stride = block_table.shape[1]
    _check(library().imparo_qk_norm_rope_store(
        _dev(qkv, "qkv", torch.float32, (n, units * head_dim)),
        _dev(q_weight, "q norm weight", torch.float32, (head_dim,)),
        _dev(k_weight, "k norm weight", torch.float32, (head_dim,)), float(eps),
        _dev(inv_freq, "inverse frequencies", torch.float32), n_freq, int(interleaved),
        _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), table_stride, page_size,
        _dev(q_out, "q out", None, (n, heads, head_dim)), _dev(k_cache, "k cache"), _dev(v_cache, "v cache"),
        _code(q_out, "q out"), int(write_kv), n, heads, kv_heads, head_dim, n_pages, int(v_transposed), _stream()),
        "qk_norm_rope_store")
    return q_out


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
              positions: torch.Tensor, row_of_token: torch.Tensor, block_table: torch.Tensor,
              scale: float, window: Optional[int], v_transposed: bool = False) -> torch.Tensor:
    """The general kernel: any page size, head sizes in steps of 16 up to 512,
    float32 or bfloat16; one wave per (token, head)."""
    n, heads, head_dim = q.shape
    n_pages, kv_heads, page_size, hd = k_cache.shape
    if hd != head_dim:
        raise KernelArgumentError(f"attention: q has head size {head_dim}, the cache {hd}")
    if head_dim % 16 != 0:
        raise KernelArgumentError(f"attention: head size must be a multiple of 16, got {head_dim}")
    if heads % kv_heads != 0:
        raise KernelArgumentError(f"attention: {heads} heads cannot share {kv_heads} kv heads evenly")
    _check(library().imparo_attention(
        _dev(q, "q"), _dev(k_cache, "k cache", q.dtype),
        _dev(v_cache, "v cache", q.dtype, (n_pages, kv_heads, head_dim, page_size) if v_transposed else k_cache.shape),
        _dev(out, "attention out", q.dtype, (n, heads * head_dim)), _code(q, "q"),
        _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size,
        n, heads, kv_heads, head_dim, n_pages, float(scale), int(window or 0), int(v_transposed), _stream()),
        "attention")
    return out


def decode_split() -> int:
    """Keys per split of the matrix-core decode kernel: its partial results hold one entry per split."""
    return int(library().imparo_attention_decode_split())


def prefill_tile() -> int:
    """Queries per tile that `attention_prefill`'s n_tiles counts."""
    return int(library().imparo_attention_prefill_tile())


def mfma_attention_supported(dtype: torch.dtype, page_size: int, head_dim: int) -> bool:
    return (dtype == torch.bfloat16 and page_size >= 16 and page_size & (page_size - 1) == 0
            and head_dim % 16 == 0 and head_dim <= 128)


def _check_mfma(q, k_cache, v_cache, out):
    n, heads, head_dim = q.shape
    n_pages, kv_heads, page_size, hd = k_cache.shape
    if not mfma_attention_supported(q.dtype, page_size, head_dim) or hd != head_dim:
        raise KernelArgumentError(f"the matrix-core attention kernels take bfloat16, pages of a power of two >= 16 and "
                                  f"head sizes in steps of 16 up to 128; got {q.dtype}, pages of {page_size}, "
                                  f"head size {head_dim}")
    if heads % kv_heads != 0:
        raise KernelArgumentError(f"attention: {heads} heads cannot share {kv_heads} kv heads evenly")
    _dev(k_cache, "k cache", torch.bfloat16)
    _dev(v_cache, "v cache", torch.bfloat16, (n_pages, kv_heads, head_dim, page_size))
    _dev(out, "attention out", torch.bfloat16, (n, heads * head_dim))
    return n, heads, head_dim, n_pages, kv_heads, page_size


def attention_decode(q, k_cache, v_cache, out, part_o, part_ml, rows, n_rows: int, seg_start, positions,
                     block_table, scale: float, window: Optional[int], max_context: int) -> torch.Tensor:
    """Split-KV attention for rows that bring one token each. `rows` lists
    them (indices into seg_start); `max_context` bounds every row's position + 1."""
    n, heads, head_dim, n_pages, kv_heads, page_size = _check_mfma(q, k_cache, v_cache, out)
    split = decode_split()
    n_splits = max(1, (max_context + split - 1) // split)
    if part_o.numel() < n_rows * heads * n_splits * head_dim or part_ml.numel() < n_rows * heads * n_splits * 2:
        raise KernelArgumentError("attention_decode: the scratch for partial results is too small")
    _check(library().imparo_attention_decode(
        _dev(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        _dev(part_o, "partial outputs", torch.float32), _dev(part_ml, "partial sums", torch.float32),
        _dev(rows, "decode rows", torch.int32), n_rows, _dev(seg_start, "seg_start", torch.int32),
        _dev(positions, "positions", torch.int32, (n,)), _dev(block_table, "block table", torch.int32),
        block_table.shape[1], page_size, heads, kv_heads, head_dim, n_pages, float(scale), int(window or 0),
        n_splits, _stream()), "attention_decode")
    return out


def attention_decode_qkv_takes(head_dim: int, n_freq: int) -> bool:
    """Whether attention_decode_qkv takes heads of this size with this many rotated pairs."""
    return bool(library().imparo_attention_decode_qkv_takes(int(head_dim), int(n_freq)))


def attention_decode_qkv_pays(n_rows: int, max_context: int) -> bool:
    """Whether the one launch is the faster way for a step of this many rows whose longest context is `max_context`."""
    n_splits = max(1, -(-int(max_context) // decode_split()))
    return bool(library().imparo_attention_decode_qkv_pays(int(n_rows), n_splits))


def attention_decode_qkv(qkv, q_weight, k_weight, eps: float, inv_freq, k_cache, v_cache, out, part_o, part_ml,
                         rows, n_rows: int, seg_start, positions, block_table, heads: int, scale: float,
                         window: Optional[int], max_context: int, interleaved: bool = False,
                         write_kv: bool = True) -> torch.Tensor:
    """qk_norm_rope_store and attention_decode in one launch less, for a step whose rows all bring one
    token: `qkv` is the fused projection's float32 rows; the new keys and values are weighed in from
    registers and, with `write_kv`, written into their pages (V pages transposed)."""
    n_pages, kv_heads, page_size, head_dim = k_cache.shape
    n = qkv.shape[0]
    _dev(qkv, "qkv", torch.float32, (n, (heads + 2 * kv_heads) * head_dim))
    _dev(out, "attention out", torch.bfloat16)
    if out.numel() != n * heads * head_dim:
        raise KernelArgumentError("attention_decode_qkv: the output does not match the rows")
    if k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16 or tuple(v_cache.shape) != (n_pages, kv_heads, head_dim, page_size):
        raise KernelArgumentError("attention_decode_qkv: bfloat16 caches, V pages transposed")
    n_freq = 0 if inv_freq is None else inv_freq.shape[0]
    if not attention_decode_qkv_takes(head_dim, n_freq):
        raise KernelArgumentError(f"attention_decode_qkv: heads of {head_dim} with {n_freq} rotated pairs are not taken")
    split = decode_split()
    n_splits = max(1, (max_context + split - 1) // split)
    if part_o.numel() < n_rows * heads * n_splits * head_dim or part_ml.numel() < n_rows * heads * n_splits * 2:
        raise KernelArgumentError("attention_decode_qkv: the scratch for partial results is too small")
    _check(library().imparo_attention_decode_qkv(
        qkv.data_ptr(), _dev(q_weight, "q norm weight", torch.float32, (head_dim,)),
        _dev(k_weight, "k norm weight", torch.float32, (head_dim,)), float(eps),
        _dev(inv_freq, "inv_freq", torch.float32), n_freq, int(bool(interleaved)), k_cache.data_ptr(),
        v_cache.data_ptr(), int(bool(write_kv)), out.data_ptr(), _dev(part_o, "partial outputs", torch.float32),
        _dev(part_ml, "partial sums", torch.float32), _dev(rows, "decode rows", torch.int32), n_rows,
        _dev(seg_start, "seg_start", torch.int32), _dev(positions, "positions", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, heads, kv_heads, head_dim,
        n_pages, float(scale), int(window or 0), n_splits, _stream()), "attention_decode_qkv")
    return out


def attention_prefill_splits(n_tiles: int, heads: int, kv_heads: int, head_dim: int, max_context: int) -> int:
    """Into how many parts the keys of a launch of prompt portions are cut (1: none): few queries
    over long contexts would leave most of the chip idle."""
    return int(library().imparo_attention_prefill_splits(n_tiles, heads, kv_heads, head_dim, max_context))


def attention_prefill(q, k_cache, v_cache, out, rows, n_rows: int, n_tiles: int, seg_start, seg_len, positions,
                      block_table, scale: float, window: Optional[int], part_o: Optional[torch.Tensor] = None,
                      part_ml: Optional[torch.Tensor] = None, n_splits: int = 1) -> torch.Tensor:
    """Tiled attention for rows that bring a portion of a prompt. `n_tiles` is
    the sum over the listed rows of ceil(seg_len / prefill_tile()). With `n_splits` > 1
    (attention_prefill_splits) each block's keys are walked in that many parts,
    merged by a second launch: `part_o` [n, heads, n_splits, head_dim] and
    `part_ml` [n, heads, n_splits, 2] float32 hold the parts."""
    n, heads, head_dim, n_pages, kv_heads, page_size = _check_mfma(q, k_cache, v_cache, out)
    if n_splits > 1:
        if part_o is None or part_ml is None:
            raise KernelArgumentError("attention_prefill: parts of the keys need buffers for their results")
        _dev(part_o, "part_o", torch.float32)
        _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < n * heads * n_splits * head_dim or part_ml.numel() < n * heads * n_splits * 2:
            raise KernelArgumentError("attention_prefill: the buffers for the parts are too small")
    _check(library().imparo_attention_prefill(
        _dev(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        part_o.data_ptr() if n_splits > 1 else None, part_ml.data_ptr() if n_splits > 1 else None, int(n_splits),
        _dev(rows, "prefill rows", torch.int32), n_rows, n_tiles, _dev(seg_start, "seg_start", torch.int32),
        _dev(seg_len, "seg_len", torch.int32), _dev(positions, "positions", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, heads, kv_heads, head_dim,
        n_pages, float(scale), int(window or 0), _stream()), "attention_prefill")
    return out


def short_conv(bcx: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
               row_of_token: torch.Tensor, seg_start: torch.Tensor, seg_len: torch.Tensor, slot: torch.Tensor,
               out: torch.Tensor, single_tokens: bool = False) -> torch.Tensor:
    """Gated short convolution of every request's segment, then the state
    update; the two launches are ordered by the stream. `single_tokens`: the
    caller knows that every request brings exactly one token; output and
    update then share one launch."""
    n, three_w = bcx.shape
    width, taps = weight.shape
    if three_w != 3 * width:
        raise KernelArgumentError(f"short_conv: rows of {three_w} values do not hold B, C and x of width {width}")
    n_slots = state.shape[0]
    n_rows = seg_start.shape[0]
    lib = library()
    if single_tokens:
        if n != n_rows:
            raise KernelArgumentError("short_conv: single_tokens needs one token per request")
        _check(lib.imparo_short_conv_decode(
            _dev(bcx, "bcx", torch.float32), _dev(weight, "conv weight", torch.float32),
            _dev(bias, "conv bias", torch.float32, (width,)),
            _dev(state, "conv state", torch.float32, (n_slots, taps - 1, width)),
            _dev(slot, "slot", torch.int32, (n_rows,)), _dev(out, "conv out", None, (n, width)), _code(out, "conv out"),
            n_rows, width, taps, n_slots, _stream()), "short_conv_decode")
        return out
    _check(lib.imparo_short_conv(
        _dev(bcx, "bcx", torch.float32), _dev(weight, "conv weight", torch.float32),
        _dev(bias, "conv bias", torch.float32, (width,)),
        _dev(state, "conv state", torch.float32, (n_slots, taps - 1, width)),
        _dev(row_of_token, "row_of_token", torch.int32, (n,)), _dev(seg_start, "seg_start", torch.int32, (n_rows,)),
        _dev(slot, "slot", torch.int32, (n_rows,)), _dev(out, "conv out", None, (n, width)), _code(out, "conv out"),
        n, width, taps, n_slots, n_rows, _stream()), "short_conv")
    _check(lib.imparo_short_conv_state(
        bcx.data_ptr(), state.data_ptr(), seg_start.data_ptr(), _dev(seg_len, "seg_len", torch.int32, (n_rows,)),
        slot.data_ptr(), n_rows, n, width, taps, n_slots, _stream()), "short_conv_state")
    return out


def in_proj_conv_decode_supported(x_rows: int, weight: torch.Tensor) -> bool:
    """The fused launch takes a bfloat16 projection and at most 16 rows."""
    return weight.dtype == torch.bfloat16 and 0 < x_rows <= 16 and weight.shape[0] % 24 == 0 and weight.shape[1] % 8 == 0


def in_proj_conv_decode(x: torch.Tensor, in_weight: torch.Tensor, in_bias: Optional[torch.Tensor],
                        conv_weight: torch.Tensor, conv_bias: Optional[torch.Tensor], state: torch.Tensor,
                        slot: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """For rows of one token each: [B | C | x] = x . in_weight^T (+ bias), then the gated short
    convolution against each row's state, which is shifted; one launch."""
    m, k = x.shape
    three_e, kw = in_weight.shape
    width, taps = conv_weight.shape
    if three_e != 3 * width or kw != k:
        raise KernelArgumentError(f"in_proj_conv_decode: a [{three_e}, {kw}] projection does not feed a conv of "
                                  f"width {width} from rows of {k}")
    if not in_proj_conv_decode_supported(m, in_weight) or x.dtype != torch.bfloat16:
        raise KernelArgumentError("in_proj_conv_decode: takes 1 to 16 bfloat16 rows and a bfloat16 projection whose "
                                  "width is a multiple of 8")
    n_slots = state.shape[0]
    _check(library().imparo_in_proj_conv_decode(
        _dev(x, "x", torch.bfloat16), _dev(in_weight, "in_proj weight", torch.bfloat16),
        _dev(in_bias, "in_proj bias", torch.float32, (three_e,)), _dev(conv_weight, "conv weight", torch.float32),
        _dev(conv_bias, "conv bias", torch.float32, (width,)),
        _dev(state, "conv state", torch.float32, (n_slots, taps - 1, width)),
        _dev(slot, "slot", torch.int32, (m,)), _dev(out, "conv out", None, (m, width)), _code(out, "conv out"),
        m, width, k, taps, n_slots, _stream()), "in_proj_conv_decode")
    return out


def rows_parts(n: int) -> int:
    """Partial sums of squares that `rows_gemm(..., into=...)` leaves for a weight of n rows."""
    return int(library().imparo_rows_parts(int(n)))


def rows_gemm(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
              swiglu: bool = False, ssq_in: Optional[torch.Tensor] = None, eps: float = 0.0,
              into: Optional[torch.Tensor] = None, ssq_out: Optional[torch.Tensor] = None,
              weighted_out: Optional[torch.Tensor] = None, weighted_by: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Products of a step of at most 16 rows with a norm of the residual stream folded in. x [m, k] and
    w [n, k] bfloat16. With `ssq_in` [parts, 16] and `eps`, x is the stream times a norm's weight and row
    r's result is multiplied by rsqrt(sum_p ssq_in[p][r] / k + eps). Stored to `out` ([m, n], or [m, n/2]
    with `swiglu`), or added to `into` [m, n] float32 in place; then `ssq_out` [rows_parts(n), 16] receives
    the partial sums of squares of the new rows and, with `weighted_by` [n], `weighted_out` [m, n]
    bfloat16 the new rows times it."""
    m, k = x.shape
    n, kw = w.shape
    if kw != k or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not 0 < m <= 16 or k % 8:
        raise KernelArgumentError("rows_gemm: 1 to 16 bfloat16 rows, a bfloat16 weight over the same inner size, "
                                  "a multiple of 8")
    n_parts = 0
    if ssq_in is not None:
        n_parts = ssq_in.shape[0]
        _dev(ssq_in, "sums of squares", torch.float32, (n_parts, 16))
    if into is not None:
        if out is not None or swiglu or ssq_out is None:
            raise KernelArgumentError("rows_gemm: adding to the stream stores nothing else and leaves sums of squares")
        _dev(into, "stream", torch.float32, (m, n))
        _dev(ssq_out, "sums of squares out", torch.float32, (rows_parts(n), 16))
        epilogue, y, code = 2, None, F32
    else:
        if out is None:
            raise KernelArgumentError("rows_gemm: an output is needed")
        _dev(out, "rows_gemm out", None, (m, n // 2 if swiglu else n))
        epilogue, y, code = int(swiglu), out, _code(out, "rows_gemm out")
    _check(library().imparo_rows_gemm(
        _dev(x, "x"), _dev(ssq_in, "sums of squares"), n_parts, float(eps), _dev(w, "weight"),
        _dev(bias, "bias", torch.float32, (n,)), _dev(y, "out"), code, _dev(into, "stream"), _dev(ssq_out, "ssq out"),
        _dev(weighted_out, "weighted out", torch.bfloat16, (m, n)), _dev(weighted_by, "weighted by", torch.float32, (n,)),
        m, n, k, epilogue, _stream()), "rows_gemm")
    return into if into is not None else out


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    n, vocab = logits.shape
    _check(library().imparo_argmax_rows(_dev(logits, "logits", torch.float32), _dev(out, "picks", torch.int32, (n,)),
                                        n, vocab, _stream()), "argmax_rows")
    return out


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
                out: torch.Tensor) -> torch.Tensor:
    n, vocab = logits.shape
    _check(library().imparo_sample_rows(
        _dev(logits, "logits", torch.float32), _dev(temperature, "temperature", torch.float32, (n,)),
        _dev(uniform, "uniform", torch.float32, (n,)), _dev(out, "picks", torch.int32, (n,)),
        n, vocab, _stream()), "sample_rows")
    return out


def fill_f32(t: torch.Tensor, value: float) -> torch.Tensor:
    _check(library().imparo_fill_f32(_dev(t, "fill target", torch.float32), float(value), t.numel(), _stream()),
           "fill_f32")
    return t


def fill_sites(base: torch.Tensor, per_slot: torch.Tensor, value: torch.Tensor, slot: int) -> None:
    """Sets one slot's row of every fixed-state site in one launch: site i's row is per_slot[i]
    float32 values at address base[i] + slot * per_slot[i] * 4 and becomes value[i] everywhere."""
    n = base.shape[0]
    _check(library().imparo_fill_sites(_dev(base, "site addresses", torch.int64, (n,)),
                                       _dev(per_slot, "site row sizes", torch.int64, (n,)),
                                       _dev(value, "site values", torch.float32, (n,)), n, int(slot), _stream()),
           "fill_sites")
