"""Grouped-query attention over the paged cache.

q = Wq h, k = Wk h, v = Wv h (one fused projection), per-head RMS norm of q
and k, rotation, k and v appended to the cache at the tokens' positions before
attention of the same batch, causal softmax attention bounded by position,
then the output projection
(/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:203-250,
/root/reference/crates/imparo-model/src/cpu_support.rs:361-445)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.pages import PagedSpec, kv_spec
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_vector
from .registry import part_class, register_part

_DEFAULT_NAMES = dict(q="q_proj", k="k_proj", v="v_proj", o="o_proj", q_norm="q_norm", k_norm="k_norm")


class Attention:
    role = "mixer"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, H, Hk, D = spec["width"], spec["heads"], spec["kv_heads"], spec["head_dim"]
        out: Declared = {
            n["q"] + ".weight": (TensorDecl((H * D, E)), "matrix"),
            n["k"] + ".weight": (TensorDecl((Hk * D, E)), "matrix"),
            n["v"] + ".weight": (TensorDecl((Hk * D, E)), "matrix"),
            n["o"] + ".weight": (TensorDecl((E, H * D)), "matrix"),
        }
        if spec.get("qk_norm") is not None:
            out[n["q_norm"] + ".weight"] = (TensorDecl((D,), "vector"), "norm")
            out[n["k_norm"] + ".weight"] = (TensorDecl((D,), "vector"), "norm")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.engine_dtype = engine_dtype
        self.v_transposed = False        # decided with the cache's page size, in cache_spec
        self.width, self.heads, self.kv_heads, self.head_dim = (spec["width"], spec["heads"], spec["kv_heads"],
                                                                spec["head_dim"])
        if self.head_dim % 16:
            raise ValueError(f"attention kernels take head sizes in steps of 16, got {self.head_dim}")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads cannot share {self.kv_heads} kv heads evenly")
        self.scale = float(spec["scale"])
        self.window: Optional[int] = spec.get("window")
        ws = [tensors[n[x] + ".weight"] for x in ("q", "k", "v")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        # one projection for q | k | v: the same dot products, one launch
        self.qkv = Linear(place_matrix(torch.cat(ws, dim=0), engine_dtype, device))
        self.out = Linear(place_matrix(tensors[n["o"] + ".weight"], engine_dtype, device))
        norm = spec.get("qk_norm")
        if norm is not None:
            # the kernels that norm a head know one norm: RMS with a weight per dimension, no offset
            if getattr(norm, "kind", "rms_norm") != "rms_norm":
                raise ValueError(f"this attention mixer norms q and k per head with an RMS norm; the plan names "
                                 f"{norm.kind!r} (another norm on the heads is another mixer, with kernels of its own)")
            self.norm_eps = float(norm["eps"])
            self.q_norm = place_vector(tensors[n["q_norm"] + ".weight"], device)
            self.k_norm = place_vector(tensors[n["k_norm"] + ".weight"], device)
        else:
            self.norm_eps, self.q_norm, self.k_norm = 0.0, None, None
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos.kind)(pos, device)
        if self.position.rotary_dim > self.head_dim:
            raise ValueError("the rotated part of a head cannot be wider than the head")

    @property
    def in_dtype(self) -> torch.dtype:
        return self.qkv.in_dtype

    def cache_spec(self, page_size: int) -> PagedSpec:
        """Keys and values per position, laid out as this mixer's kernels read
        them: where the matrix-core kernels apply (bfloat16, pages of at least
        16, head sizes up to 128), V is kept transposed inside a page."""
        self.v_transposed = ops.mfma_attention_supported(self.engine_dtype, page_size, self.head_dim)
        return kv_spec(self.kv_heads, self.head_dim, self.window, self.v_transposed)

    def _portion_tiles(self, ctx: StepContext) -> int:
        """Tiles of queries that the portions of this batch make, as the prompt kernel counts them."""
        key = ("attention portion tiles", ops.prefill_tile())
        if key not in ctx.memo:
            tile = ops.prefill_tile()
            ctx.memo[key] = sum((int(n) + tile - 1) // tile for n in ctx.host_seg_len if n > 1)
        return ctx.memo[key]

    def _decode_parts(self, ctx: StepContext):
        """Room for the partial results of the single-token rows' splits."""
        split = ops.decode_split()
        n_splits = (ctx.max_context + split - 1) // split
        part_o = ctx.workspace.get("attn_part_o", (ctx.n_single_rows * self.heads * n_splits * self.head_dim,),
                                   torch.float32)
        part_ml = ctx.workspace.get("attn_part_ml", (ctx.n_single_rows * self.heads * n_splits * 2,), torch.float32)
        return part_o, part_ml

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        T = h.shape[0]
        qkv = self.qkv(ctx, h, torch.float32, "qkv", alias="mixer_in")
        k_cache, v_cache, table = ctx.kv(site)
        vt = self.v_transposed
        inv_freq = self.position.inv_freq
        interleaved = bool(getattr(self.position, "interleaved", False))
        if (vt and owns_cache and ctx.single_rows is not None and ctx.n_single_rows == T and not ctx.n_portion_rows
                and ops.attention_decode_qkv_pays(T, ctx.max_context)
                and ops.attention_decode_qkv_takes(self.head_dim, 0 if inv_freq is None else inv_freq.shape[0])):
            # every row brings one token: head norm, rotation and the write of the new key and value ride
            # in the attention launch (the new key is weighed in from registers)
            o = ctx.workspace.get("attn_out", (T, self.heads * self.head_dim), ctx.dtype, alias="mixer_mid")
            part_o, part_ml = self._decode_parts(ctx)
            ops.attention_decode_qkv(qkv, self.q_norm, self.k_norm, self.norm_eps, inv_freq, k_cache, v_cache, o,
                                     part_o, part_ml, ctx.single_rows, ctx.n_single_rows, ctx.seg_start,
                                     ctx.positions, table, self.heads, self.scale, self.window, ctx.max_context,
                                     interleaved=interleaved)
            return self.out(ctx, o, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)
        q = ctx.workspace.get("q", (T, self.heads, self.head_dim), ctx.dtype)
        ops.qk_norm_rope_store(qkv, self.q_norm, self.k_norm, self.norm_eps, inv_freq,
                               ctx.positions, ctx.row_of_token, table if owns_cache else None, ctx.page_size,
                               q, k_cache if owns_cache else None, v_cache if owns_cache else None,
                               self.heads, self.kv_heads, self.head_dim, v_transposed=vt, interleaved=interleaved)
        o = ctx.workspace.get("attn_out", (T, self.heads * self.head_dim), ctx.dtype, alias="mixer_mid")
        if vt and ctx.single_rows is not None:
            # matrix-core kernels: single tokens split over their keys, portions tiled over their queries
            if ctx.n_single_rows:
                part_o, part_ml = self._decode_parts(ctx)
                ops.attention_decode(q, k_cache, v_cache, o, part_o, part_ml, ctx.single_rows, ctx.n_single_rows,
                                     ctx.seg_start, ctx.positions, table, self.scale, self.window, ctx.max_context)
            if ctx.n_portion_rows:
                # few queries over long contexts: each block's keys in parts, merged by a second launch
                n_tiles = self._portion_tiles(ctx)
                # (the bound on the contexts that the launch itself sees: what its block table can hold)
                parts = ops.attention_prefill_splits(n_tiles, self.heads, self.kv_heads, self.head_dim,
                                                     table.shape[1] * ctx.page_size)
                part_o = part_ml = None
                if parts > 1:
                    part_o = ctx.workspace.get("attn_prefill_part_o", (T * self.heads * parts * self.head_dim,),
                                               torch.float32)
                    part_ml = ctx.workspace.get("attn_prefill_part_ml", (T * self.heads * parts * 2,), torch.float32)
                ops.attention_prefill(q, k_cache, v_cache, o, ctx.portion_rows, ctx.n_portion_rows,
                                      n_tiles, ctx.seg_start, ctx.seg_len, ctx.positions, table,
                                      self.scale, self.window, part_o, part_ml, parts)
        else:
            ops.attention(q, k_cache, v_cache, o, ctx.positions, ctx.row_of_token, table, self.scale, self.window,
                          v_transposed=vt)
        if o.dtype != self.out.in_dtype:
            raise ValueError("the output projection's weight dtype differs from the attention output's")
        # a delta for the residual stream: the next norm adds slices, so it may come sliced
        return self.out(ctx, o, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


    def emit(self, program, site: int, owns_cache: bool) -> None:
        """Appends `forward` to a native step program."""
        from ..kernels.program import AttentionDesc
        arrays = program.storage.paged[site]
        k_cache, v_cache = arrays["k"], arrays["v"]
        inv_freq = self.position.inv_freq
        program.attention(AttentionDesc(
            program.linear(self.qkv), program.linear(self.out),
            program._hold(self.q_norm, "q norm weight", torch.float32),
            program._hold(self.k_norm, "k norm weight", torch.float32), self.norm_eps,
            program._hold(inv_freq, "inverse frequencies", torch.float32), 0 if inv_freq is None else inv_freq.shape[0],
            int(bool(getattr(self.position, "interleaved", False))), self.heads, self.kv_heads, self.head_dim,
            self.scale, int(self.window or 0), program._hold(k_cache, "k cache"), program._hold(v_cache, "v cache"),
            k_cache.shape[0], int(self.v_transposed), program.group_of_site[site], int(owns_cache)))


register_part("mixer", "attention", Attention)
