"""How a layer's parts are arranged.

pre_norm: x += mixer(norm_a(x)); x += ffn(norm_b(x)) -- no post-norms
(/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:8-15). Each
delta is left pending on the residual stream so that the next norm, whichever
block it belongs to, adds it while reading the row."""
from __future__ import annotations

from typing import Dict

from .base import Residual, StepContext, emits
from .registry import register_part


class PreNormBlock:
    """Reads four parts by name: mixer_norm, mixer, ffn_norm, ffn."""
    role = "block"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    def __init__(self, parts: Dict[str, object]):
        self.parts = parts
        self.mixer_norm, self.mixer = parts["mixer_norm"], parts["mixer"]
        self.ffn_norm, self.ffn = parts["ffn_norm"], parts["ffn"]

    def cache_spec(self, page_size: int):
        """What a call of this block keeps between steps: its mixer's state."""
        return self.mixer.cache_spec(page_size)

    def forward(self, ctx: StepContext, res: Residual, site: int, owns_cache: bool) -> None:
        h = self.mixer_norm.forward(ctx, res, self.mixer.in_dtype)
        res.pending = self._delta(ctx, res, lambda: self.mixer.forward(ctx, site, owns_cache, h))
        n = self.ffn_norm.forward(ctx, res, self.ffn.in_dtype)
        res.pending = self._delta(ctx, res, lambda: self.ffn.forward(ctx, n))

    def can_emit(self) -> bool:
        return all(emits(p) for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn))

    def emit(self, program, site: int, owns_cache: bool) -> None:
        """Appends `forward` to a native step program: the four parts in the order they run."""
        self.mixer_norm.emit(program, self.mixer.in_dtype)
        self.mixer.emit(program, site, owns_cache)
        self.ffn_norm.emit(program, self.ffn.in_dtype)
        self.ffn.emit(program)

    @staticmethod
    def _delta(ctx: StepContext, res: Residual, run):
        """Runs a part whose result goes into the stream. With nothing pending the part may add its
        result to the stream itself (it then returns the stream); otherwise it returns a delta."""
        ctx.stream = res.x if res.pending is None else None
        try:
            delta = run()
        finally:
            ctx.stream = None
        return None if delta is res.x else delta


register_part("block", "pre_norm", PreNormBlock)
