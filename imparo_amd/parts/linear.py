"""A dense projection y = x . W^T (+ b) on the GEMM kernels.

Not a part of its own: mixers, feed-forwards and the head are made of these.
The weight decides the kernel: a bfloat16 weight runs the MFMA kernels, a
float32 weight the float32 kernel; the input must already be in that dtype
(`in_dtype`), which the producer of the input asks for.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import StepContext


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2:
            raise ValueError(f"a projection weight is [out, in], got shape {list(weight.shape)}")
        self.weight = weight.contiguous()
        self.bias = None if bias is None else bias.to(torch.float32).contiguous()
        self.out_features, self.in_features = weight.shape

    @property
    def in_dtype(self) -> torch.dtype:
        return self.weight.dtype

    def __call__(self, ctx: StepContext, x: torch.Tensor, out_dtype: torch.dtype, name: str,
                 swiglu: bool = False, sliced_ok: bool = False, alias: Optional[str] = None,
                 into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """`swiglu`: the weight's rows alternate gate and up; the output is
        silu(gate) * up, half as wide. `sliced_ok`: the caller's consumer adds
        slices, so the result may come as [slices, rows, out] sums over parts
        of K (few rows and a long K keep more of the chip busy that way).
        `alias`: the workspace group the output may share memory with.
        `into`: a float32 [rows, out] tensor the result may be added to instead
        (the residual stream); where the kernels do that, `into` itself is returned."""
        width = self.out_features // 2 if swiglu else self.out_features
        m = x.shape[0]
        if sliced_ok and not swiglu and out_dtype == torch.float32:
            slices = ops.gemm_slices(m, self.out_features, self.in_features, self.weight.dtype)
            if slices > 1:
                out = ctx.workspace.get(name + "_sliced", (slices, m, width), out_dtype)
                return ops.gemm(x, self.weight, out, bias=self.bias)
        if (into is not None and not swiglu and out_dtype == torch.float32 and into.dtype == torch.float32
                and tuple(into.shape) == (m, width) and into.is_contiguous()
                and ops.gemm_adds(m, self.out_features, self.in_features, self.weight.dtype)):
            # one pass less over the rows for the norm that follows: the product's epilogue reads and writes the stream
            return ops.gemm(x, self.weight, into, bias=self.bias, add=True)
        out = ctx.workspace.get(name, (m, width), out_dtype, alias=alias)
        return ops.gemm(x, self.weight, out, bias=self.bias, swiglu=swiglu)


def place_matrix(t: torch.Tensor, engine_dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """A matrix as the engine keeps it on the device: bfloat16 stays bfloat16
    under a bfloat16 engine, everything is float32 under a float32 engine, and
    a tensor stored in float32 stays float32 either way."""
    if engine_dtype == torch.float32 or t.dtype == torch.float32:
        return t.to(device=device, dtype=torch.float32).contiguous()
    return t.to(device=device, dtype=torch.bfloat16).contiguous()


def place_vector(t: torch.Tensor, device: torch.device) -> torch.Tensor:
    """Norm weights, conv taps and biases are read as float32 by the kernels;
    widening bfloat16 to float32 is exact."""
    return t.to(device=device, dtype=torch.float32).contiguous()
