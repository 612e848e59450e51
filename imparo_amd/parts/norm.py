"""RMS norm: y = x * rsqrt(mean(x^2) + eps) * w, no offset, no bias
(/root/reference/crates/imparo-cpu/src/ops.rs:6-22). The residual add that
precedes a norm is fused into it (the reference's add_rms_norm,
/root/reference/crates/imparo-backend/src/lib.rs:2603-2609)."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, Residual, StepContext
from .linear import place_vector
from .registry import register_part


class RmsNorm:
    role = "norm"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def declare(spec: PartSpec) -> Declared:
        return {f"{spec.prefix}.weight": (TensorDecl((spec["width"],), "vector"), "norm")}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        self.width = spec["width"]
        self.eps = float(spec["eps"])
        self.weight = place_vector(tensors[f"{spec.prefix}.weight"], device)

    def forward(self, ctx: StepContext, res: Residual, out_dtype: torch.dtype, name: str = "normed") -> torch.Tensor:
        """Adds the pending delta into the stream (if any) and returns the
        normed rows in `out_dtype`."""
        out = ctx.workspace.get(name, tuple(res.x.shape), out_dtype)
        if res.pending is not None:
            ops.rms_norm(res.x, self.weight, self.eps, out, delta=res.pending, write_back=True)
            res.pending = None
        else:
            ops.rms_norm(res.x, self.weight, self.eps, out)
        return out

    def emit(self, program, out_dtype: torch.dtype) -> None:
        """Appends `forward` to a native step program."""
        program.norm(self.weight, self.eps, self.width, out_dtype)

    def emit_head(self, program, head_linear) -> None:
        """Appends `forward_rows` followed by the head's projection."""
        program.head(self.weight, self.eps, self.width, head_linear)

    def forward_rows(self, ctx: StepContext, res: Residual, rows: torch.Tensor, out_dtype: torch.dtype,
                     name: str = "normed_rows") -> torch.Tensor:
        """Norm of selected rows only (the rows whose logits are wanted); the
        stream itself is left as it is."""
        out = ctx.workspace.get(name, (rows.shape[0], self.width), out_dtype)
        ops.rms_norm(res.x, self.weight, self.eps, out, delta=res.pending, rows=rows)
        return out


register_part("norm", "rms_norm", RmsNorm)
