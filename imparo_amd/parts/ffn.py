"""Dense SwiGLU feed-forward: f = W2 ( silu(W1 n) * (W3 n) ), SiLU on the gate
(/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:298-316)."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.plan import PartSpec
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix
from .registry import register_part

_DEFAULT_NAMES = dict(gate="gate_proj", up="up_proj", down="down_proj")


class SwiGlu:
    role = "feed_forward"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, F = spec["width"], spec["hidden"]
        return {
            n["gate"] + ".weight": (TensorDecl((F, E)), "matrix"),
            n["up"] + ".weight": (TensorDecl((F, E)), "matrix"),
            n["down"] + ".weight": (TensorDecl((E, F)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.hidden = spec["width"], spec["hidden"]
        gate, up = tensors[n["gate"] + ".weight"], tensors[n["up"] + ".weight"]
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        down = tensors[n["down"] + ".weight"]
        # The bfloat16 kernels walk K in steps of 8. A hidden width that is no multiple of 8 is
        # filled up with hidden units whose weights are zero: silu(0) * 0 = 0 goes through zero
        # columns of the way back, so every sum is the one it was.
        fill = (-self.hidden) % 8
        if fill and engine_dtype != torch.float32 and down.dtype != torch.float32:
            gate = torch.cat([gate, gate.new_zeros(fill, self.width)])
            up = torch.cat([up, up.new_zeros(fill, self.width)])
            down = torch.cat([down, down.new_zeros(self.width, fill)], dim=1)
        # gate and up as one projection with alternating rows (g0, u0, g1, u1, ...): the same dot
        # products, one launch, and the GEMM's epilogue applies silu(gate) * up before it stores
        fused = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], self.width)
        self.gate_up = Linear(place_matrix(fused, engine_dtype, device))
        self.down = Linear(place_matrix(down, engine_dtype, device))

    @property
    def in_dtype(self) -> torch.dtype:
        return self.gate_up.in_dtype

    def forward(self, ctx: StepContext, n: torch.Tensor) -> torch.Tensor:
        # the gated hidden may lie where the mixer's input projection lay: that is dead by now
        g = self.gate_up(ctx, n, self.down.in_dtype, "gated", swiglu=True, alias="mixer_in")
        # the result is a delta for the residual stream, whose next norm adds slices: it may come sliced
        return self.down(ctx, g, torch.float32, "ffn_out", sliced_ok=True, into=ctx.stream)


    def emit(self, program) -> None:
        """Appends `forward` to a native step program."""
        from ..kernels.program import SwigluDesc
        program.swiglu(SwigluDesc(program.linear(self.gate_up), program.linear(self.down)))


register_part("feed_forward", "swiglu", SwiGlu)
