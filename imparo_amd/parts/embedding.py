"""Token embedding (a row gather, no scale:
/root/reference/crates/imparo-model/src/cpu_support.rs:327-342) and the output
head (logits = W h for the rows that want logits, no bias, no softcap:
/root/reference/crates/imparo-model/src/cpu_support.rs:451-466)."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix
from .registry import register_part


class Embedding:
    role = "embedding"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def declare(spec: PartSpec) -> Declared:
        return {f"{spec.prefix}.weight": (TensorDecl((spec["vocab"], spec["width"])), "matrix")}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype, placed: Dict[str, torch.Tensor]):
        name = f"{spec.prefix}.weight"
        if name not in placed:     # a tied head shares this very tensor
            placed[name] = place_matrix(tensors[name], engine_dtype, device)
        self.table = placed[name]
        self.vocab, self.width = spec["vocab"], spec["width"]

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        x = ctx.workspace.get("residual", (token_ids.shape[0], self.width), torch.float32)
        return ops.embed_gather(self.table, token_ids, x)

    def emit(self, program) -> None:
        """Appends `forward` to a native step program."""
        program.embedding(self.table, self.vocab, self.width)


class LinearHead:
    role = "head"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def declare(spec: PartSpec) -> Declared:
        return {f"{spec.prefix}.weight": (TensorDecl((spec["vocab"], spec["width"])), "matrix")}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype, placed: Dict[str, torch.Tensor]):
        name = f"{spec.prefix}.weight"
        if name not in placed:
            placed[name] = place_matrix(tensors[name], engine_dtype, device)
        self.proj = Linear(placed[name])
        self.vocab = spec["vocab"]

    @property
    def in_dtype(self) -> torch.dtype:
        return self.proj.in_dtype

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        return self.proj(ctx, h, torch.float32, "logits")

    def emit_projection(self) -> Linear:
        """What `forward` computes, for a native step program: this projection, float32 out."""
        return self.proj


register_part("embedding", "embedding", Embedding)
register_part("head", "linear_head", LinearHead)
