"""What every part sees of a step, and small shared pieces.

StepContext is the whole interface between the step function and the parts: a
part never learns which model it is in, which request a token belongs to
beyond its row, or how the batch was cut.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from ..weights.loader import TensorDecl

# (declaration, how random-weights mode initialises it: "matrix" | "conv" | "norm" | "bias")
Declared = Dict[str, Tuple[TensorDecl, str]]


class Workspace:
    """Named scratch tensors that live across steps, so a step allocates
    nothing once sizes have been seen. Kernels of one step run in order on one
    stream, so a name can be reused by every layer."""

    def __init__(self, device: torch.device):
        self.device = device
        self._buffers: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}

    def get(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= s
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
        return buf[:n].view(shape)


@dataclass
class StepContext:
    """One batch as the parts see it. All tensors are int32 on the device.

    token t of the packed batch belongs to request row `row_of_token[t]` and
    sits at absolute position `positions[t]`; row r's tokens are
    [seg_start[r], seg_start[r] + seg_len[r]) and its fixed state lives in
    slot `slot[r]`; `block_tables[g]` is [rows, pages] for cache group g.
    """
    n_tokens: int
    n_rows: int
    positions: torch.Tensor
    row_of_token: torch.Tensor
    seg_start: torch.Tensor
    seg_len: torch.Tensor
    slot: torch.Tensor
    block_tables: Dict[int, torch.Tensor]
    page_size: int
    dtype: torch.dtype                  # activation / cache dtype of this engine
    workspace: Workspace
    storage: "object"                   # imparo_amd.cache.storage.CacheStorage
    group_of_site: Dict[int, int]
    max_seg_len: int = 1                # host copy: longest segment of the batch
    max_context: int = 0                # host copy: longest context after this step
    # rows that bring one token / more than one, as index lists into seg_start
    decode_rows: Optional[torch.Tensor] = None
    n_decode_rows: int = 0
    prefill_rows: Optional[torch.Tensor] = None
    n_prefill_rows: int = 0
    n_prefill_tiles: int = 0            # sum over prefill rows of ceil(seg_len / 64)

    def kv(self, site: int):
        k, v = self.storage.kv[site]
        return k, v, self.block_tables[self.group_of_site[site]]

    def v_transposed(self, site: int) -> bool:
        return bool(getattr(self.storage, "v_transposed", {}).get(site, False))

    def fixed_state(self, site: int) -> torch.Tensor:
        return self.storage.fixed[site]


@dataclass
class Residual:
    """The residual stream in float32 and a delta not yet added to it. The
    next norm adds the delta while it reads the row anyway. The delta is
    shaped like x, or [slices, *x.shape]: sums over parts of a projection's
    inner dimension, which the norm adds up in order."""
    x: torch.Tensor
    pending: Optional[torch.Tensor] = None
