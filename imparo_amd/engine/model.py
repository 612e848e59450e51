"""Plan + weights -> a runnable stack of parts.

The builder knows roles and registries, not architectures: every layer's
norms, mixer and feed-forward are looked up by the kind its PartSpec names and
built from the tensors they declared. The run order is the plan's list of
calls; each call that owns a cache gets a cache site of its own, a call that
reads another call's cache is bound to that call's site.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.pages import StateSpec
from ..config.plan import ModelPlan, PartSpec
from ..parts import part_class
from ..parts.base import Declared, Residual, StepContext, emits


def _declare(role: str, spec: PartSpec) -> Declared:
    return part_class(role, spec.kind).declare(spec)


def declared_tensors(plan: ModelPlan) -> Declared:
    """Every tensor the model reads, by name: what the parts declare, united.
    A name two parts declare (a tied head) must agree in shape."""
    out: Declared = {}

    def add(d: Declared) -> None:
        for name, (decl, init) in d.items():
            if name in out and out[name][0].shape != decl.shape:
                raise ValueError(f"tensor {name} is declared with shapes {out[name][0].shape} and {decl.shape}")
            out[name] = (decl, init)

    add(_declare("embedding", plan.embedding))
    for layer in plan.layers:
        for role, spec in layer.parts.values():
            add(_declare(role, spec))
    add(_declare("norm", plan.final_norm))
    add(_declare("head", plan.head))
    return out


class Model:
    def __init__(self, plan: ModelPlan, tensors: Dict[str, torch.Tensor], device: torch.device,
                 dtype: torch.dtype, page_size: int):
        plan.validate()
        self.plan = plan
        self.device = device
        self.dtype = dtype
        placed: Dict[str, torch.Tensor] = {}
        self.embedding = part_class("embedding", plan.embedding.kind)(plan.embedding, tensors, device, dtype, placed)
        self.blocks = []
        built = []
        for layer in plan.layers:
            parts = {name: part_class(role, spec.kind)(spec, tensors, device, dtype)
                     for name, (role, spec) in layer.parts.items()}
            built += list(parts.values())
            self.blocks.append(part_class("block", layer.arrangement)(parts))
        self.final_norm = part_class("norm", plan.final_norm.kind)(plan.final_norm, tensors, device, dtype)
        self.head = part_class("head", plan.head.kind)(plan.head, tensors, device, dtype, placed)
        # a step can be captured into a graph only if every part says it launches kernels and nothing else
        self.graph_safe = all(getattr(p, "graph_safe", False)
                              for p in [self.embedding, self.final_norm, self.head] + self.blocks + built)
        # cache sites: one per entry of the run order; None where the call borrows
        self.site_of_call: List[int] = []
        self.site_specs: List[StateSpec] = []
        for i, call in enumerate(plan.order):
            spec = self.blocks[call.layer].cache_spec(page_size)
            if call.cache_of is None:
                self.site_of_call.append(i)
                self.site_specs.append(spec)
            else:
                self.site_of_call.append(call.cache_of)
                self.site_specs.append(None)
                owner = self.site_specs[call.cache_of]
                if owner != spec:
                    raise ValueError(f"run order entry {i} reads the cache of entry {call.cache_of}, "
                                     f"whose state has another shape")

    def forward(self, ctx: StepContext, token_ids: torch.Tensor, want_rows: Optional[torch.Tensor]
                ) -> Optional[torch.Tensor]:
        """Runs the batch through every call of the order. Returns float32
        logits [wanted, vocab] for `want_rows` (indices into the packed
        batch), or None if nothing is wanted; the head is skipped then."""
        res = Residual(self.embedding.forward(ctx, token_ids))
        for i, call in enumerate(self.plan.order):
            self.blocks[call.layer].forward(ctx, res, self.site_of_call[i], call.cache_of is None)
        if want_rows is None or want_rows.shape[0] == 0:
            return None
        h = self.final_norm.forward_rows(ctx, res, want_rows, self.head.in_dtype)
        return self.head.forward(ctx, h)

    def build_program(self, storage, group_of_site: Dict[int, int], page_size: int):
        """The run order as a native step program (one call issues a step's
        kernels), or None if some part cannot append itself to one: a part
        registered from outside, say; the parts then run one by one."""
        from ..kernels.program import MAX_GROUPS, Program
        if len(set(group_of_site.values())) > MAX_GROUPS:
            return None
        blocks_emit = all(emits(b) and getattr(b, "can_emit", lambda: True)() for b in self.blocks)
        if not (blocks_emit and emits(self.embedding) and emits(self.final_norm, "emit_head", "forward_rows")
                and emits(self.head, "emit_projection")):
            return None
        program = Program(self.dtype, page_size, storage, group_of_site)
        self.embedding.emit(program)
        for i, call in enumerate(self.plan.order):
            self.blocks[call.layer].emit(program, self.site_of_call[i], call.cache_of is None)
        self.final_norm.emit_head(program, self.head.emit_projection())
        return program

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        def walk(obj):
            nonlocal total
            for v in vars(obj).values():
                if isinstance(v, torch.Tensor):
                    if v.data_ptr() not in seen:
                        seen.add(v.data_ptr())
                        total += v.numel() * v.element_size()
                elif hasattr(v, "__dict__") and not isinstance(v, type):
                    walk(v)
        walk(self.embedding); walk(self.final_norm); walk(self.head)
        for b in self.blocks:
            walk(b)
        return total
