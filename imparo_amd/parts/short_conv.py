"""Gated short convolution with a fixed-size rolling state per request.

bcx = Win h, row = [B | C | x]; u = B*x; seq = state ++ u; conv_t = sum_k
w[ch,k] seq[t+k] (tap 0 is the oldest); y = C * conv; state' = last taps-1
rows of seq; m = Wout y
(/root/reference/crates/imparo-cpu/src/ops.rs:80-167,
/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:252-278).
With `bias` every projection and the conv carry one; the conv's is added
before the C gate."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.pages import FixedSpec
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_vector
from .registry import register_part


class ShortConv:
    role = "mixer"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def declare(spec: PartSpec) -> Declared:
        E, L, p = spec["width"], spec["taps"], spec.prefix
        out: Declared = {
            f"{p}.in_proj.weight": (TensorDecl((3 * E, E)), "matrix"),
            f"{p}.conv.weight": (TensorDecl((E, 1, L), "vector"), "conv"),
            f"{p}.out_proj.weight": (TensorDecl((E, E)), "matrix"),
        }
        if spec.get("bias"):
            out[f"{p}.in_proj.bias"] = (TensorDecl((3 * E,), "vector"), "bias")
            out[f"{p}.conv.bias"] = (TensorDecl((E,), "vector"), "bias")
            out[f"{p}.out_proj.bias"] = (TensorDecl((E,), "vector"), "bias")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        E, L, p = spec["width"], spec["taps"], spec.prefix
        if L < 2:
            raise ValueError("a short conv needs at least 2 taps to carry state")
        if L > 64:
            raise ValueError(f"the conv kernels take at most 64 taps, got {L}")
        self.width, self.taps = E, L
        bias = bool(spec.get("bias"))
        b = (lambda name: place_vector(tensors[f"{p}.{name}.bias"], device)) if bias else (lambda name: None)
        self.in_proj = Linear(place_matrix(tensors[f"{p}.in_proj.weight"], engine_dtype, device), b("in_proj"))
        self.out_proj = Linear(place_matrix(tensors[f"{p}.out_proj.weight"], engine_dtype, device), b("out_proj"))
        self.conv_weight = place_vector(tensors[f"{p}.conv.weight"].reshape(E, L), device)
        self.conv_bias = b("conv")

    @property
    def in_dtype(self) -> torch.dtype:
        return self.in_proj.in_dtype

    def cache_spec(self, page_size: int) -> FixedSpec:
        return FixedSpec((self.taps - 1, self.width))

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        if not owns_cache:
            raise ValueError("a short conv's state cannot be read from another layer")
        T = h.shape[0]
        y = ctx.workspace.get("conv_out", (T, self.width), self.out_proj.in_dtype, alias="mixer_mid")
        if ctx.max_seg_len == 1 and ops.in_proj_conv_decode_supported(T, self.in_proj.weight):
            # a decode step's few rows: projection and conv in one launch
            ops.in_proj_conv_decode(h, self.in_proj.weight, self.in_proj.bias, self.conv_weight, self.conv_bias,
                                    ctx.fixed_state(site), ctx.slot, y)
            return self.out_proj(ctx, y, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)
        bcx = self.in_proj(ctx, h, torch.float32, "bcx", alias="mixer_in")
        ops.short_conv(bcx, self.conv_weight, self.conv_bias, ctx.fixed_state(site), ctx.row_of_token,
                       ctx.seg_start, ctx.seg_len, ctx.slot, y, single_tokens=ctx.max_seg_len == 1)
        # a delta for the residual stream: the next norm adds slices, so it may come sliced
        return self.out_proj(ctx, y, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


    def emit(self, program, site: int, owns_cache: bool) -> None:
        """Appends `forward` to a native step program."""
        from ..kernels.program import ShortConvDesc
        if not owns_cache:
            raise ValueError("a short conv's state cannot be read from another layer")
        state = program.storage.fixed[site]
        program.short_conv(ShortConvDesc(
            program.linear(self.in_proj), program.linear(self.out_proj),
            program._hold(self.conv_weight, "conv weight", torch.float32),
            program._hold(self.conv_bias, "conv bias", torch.float32),
            self.width, self.taps, program._hold(state, "conv state", torch.float32), state.shape[0]))


register_part("mixer", "short_conv", ShortConv)
