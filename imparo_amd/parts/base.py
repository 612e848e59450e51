"""What every part sees of a step, and small shared pieces.

StepContext is the whole interface between the step function and the parts: a
part never learns which model it is in, which request a token belongs to
beyond its row, or how the batch was cut.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Sequence, Tuple

import torch

from ..weights.loader import TensorDecl

# (declaration, how random-weights mode initialises it: "matrix" | "conv" | "norm" | "bias")
Declared = Dict[str, Tuple[TensorDecl, str]]


class Workspace:
    """Named scratch tensors that live across steps, so a step allocates
    nothing once sizes have been seen. Kernels of one step run in order on one
    stream, so a name can be reused by every layer.

    Buffers never move: a name that needs more room gets a new buffer (at
    least twice the old size) and the old one stays alive as long as a
    captured step that was recorded with it does (`pin`), so every captured
    shape can share this one workspace. Names that are never live at the same
    time may share memory: `alias` names the group they share, which is as
    large as its largest member (a layer's attention scratch and its conv
    scratch; what a mixer used and what the feed-forward after it uses). The
    reference plans its activation buffers the same way, in alias groups that
    follow a block's order of work
    (/root/reference/crates/imparo-model/src/lfm2/workflow_gpu.rs:110-183)."""

    def __init__(self, device: torch.device):
        self.device = device
        self._buffers: Dict[str, torch.Tensor] = {}      # by name or alias group: raw bytes
        self.version = 0                                 # counts new buffers: who keeps addresses looks here

    def reserve(self, key: str, nbytes: int) -> torch.Tensor:
        """Makes the buffer of a name (or alias group) at least `nbytes` large and returns it."""
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < nbytes:
            grown = nbytes if buf is None else max(nbytes, 2 * buf.numel())
            buf = torch.empty((max(grown, 1) + 255) // 256 * 256, dtype=torch.uint8, device=self.device)
            self._buffers[key] = buf
            self.version += 1
        return buf

    def buffer(self, key: str) -> Optional[torch.Tensor]:
        """The buffer of a name or alias group as it is now, or None."""
        return self._buffers.get(key)

    def get(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype, alias: Optional[str] = None) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= s
        need = max(n, 1) * _ELEMENT_SIZE[dtype]
        key = alias or name
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < need:
            buf = self.reserve(key, need)
        return buf[:n * _ELEMENT_SIZE[dtype]].view(dtype).view(shape)

    def pin(self) -> list:
        """The buffers as they are now, to be kept by whoever recorded their addresses."""
        return list(self._buffers.values())

    def bytes(self) -> int:
        return sum(b.numel() for b in self._buffers.values())


_ELEMENT_SIZE = {torch.float32: 4, torch.bfloat16: 2, torch.int32: 4, torch.float16: 2, torch.int64: 8,
                 torch.uint8: 1}


@dataclass
class StepContext:
    """One batch as the parts see it. All tensors are int32 on the device.

    token t of the packed batch belongs to request row `row_of_token[t]` and
    sits at absolute position `positions[t]`; row r's tokens are
    [seg_start[r], seg_start[r] + seg_len[r]) and its fixed state lives in
    slot `slot[r]`; `block_tables[g]` is [rows, pages] for cache group g.
    `single_rows` lists the rows that bring one token, `portion_rows` those
    that bring more (indices into seg_start). `host_seg_len` is seg_len on the
    host, for parts whose launches depend on it; a captured step has none
    beyond "every row brings one token".
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
    max_context: int = 0                # host copy: longest context after this step (a captured step: its bound)
    single_rows: Optional[torch.Tensor] = None
    n_single_rows: int = 0
    portion_rows: Optional[torch.Tensor] = None
    n_portion_rows: int = 0
    host_seg_len: Optional[Sequence[int]] = None
    memo: Dict[object, object] = field(default_factory=dict)   # what parts derive from the batch, once a step
    # The float32 residual stream while a block runs the part whose result goes into it, with nothing pending
    # on it: the part may add its result there itself and return the stream instead of a delta. None: return a delta.
    stream: Optional[torch.Tensor] = None

    def paged(self, site: int):
        """The site's paged arrays by name, and the block table of its group."""
        return self.storage.paged[site], self.block_tables[self.group_of_site[site]]

    def kv(self, site: int):
        arrays, table = self.paged(site)
        return arrays["k"], arrays["v"], table

    def fixed_state(self, site: int) -> torch.Tensor:
        """The site's fixed-size state [slots, *shape]: its one array, or the one named "state"."""
        return self.storage.fixed[site]

    def fixed_arrays(self, site: int) -> Dict[str, torch.Tensor]:
        """Every array of the site's fixed-size state by name, each [slots, *shape] in its own dtype."""
        return self.storage.fixed_arrays[site]


def emits(part, emit: str = "emit", forward: str = "forward") -> bool:
    """Whether a part can append itself to a native step program: it has the
    method `emit`, and no class below the one that defines it has replaced
    `forward`, the method it describes (a subclass that computes something
    else must not inherit the description of what its parent computes)."""
    owner_of = lambda name: next((i for i, c in enumerate(type(part).__mro__) if name in c.__dict__), None)
    e, f = owner_of(emit), owner_of(forward)
    return e is not None and (f is None or e <= f)


@dataclass
class Residual:
    """The residual stream in float32 and a delta not yet added to it. The
    next norm adds the delta while it reads the row anyway. The delta is
    shaped like x, or [slices, *x.shape]: sums over parts of a projection's
    inner dimension, which the norm adds up in order."""
    x: torch.Tensor
    pending: Optional[torch.Tensor] = None
