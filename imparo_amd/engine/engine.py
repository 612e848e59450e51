"""The engine: a model folder -> one step function over a paged cache.

`step` takes a batch of (request, its next tokens, the places whose logits
are wanted): portions of prompts beside single decoded tokens, cut anywhere.
It runs only those tokens, as one batch, from the cache earlier steps left,
and returns the logits at the wanted places. A step is atomic: if it cannot
get its pages nothing changes. The reference runs either one request's chunk
or a set of single-token rows per forward
(/root/reference/crates/imparo-model/src/lib.rs:1131-1156); here both ride in
one batch.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pages import CacheManager, OutOfPages
from ..cache.storage import CacheStorage
from ..config import plan_from_config, read_config_json
from ..kernels import library
from ..parts.base import StepContext, Workspace
from ..weights import load_weights
from .model import Model, declared_tensors

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


class StepError(ValueError):
    """A batch the step function refuses; nothing has changed."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()       # places among `tokens` whose logits are wanted


class _Upload:
    """Ring of pinned host buffers + one device buffer per ring entry for the
    per-step index arrays: one copy per step, no allocation once sized."""

    def __init__(self, device: torch.device, depth: int = 4):
        self.device = device
        self.depth = depth
        self.host: List[Optional[torch.Tensor]] = [None] * depth
        self.dev: List[Optional[torch.Tensor]] = [None] * depth
        self.events: List[Optional[torch.cuda.Event]] = [None] * depth
        self.turn = 0

    def send(self, packed: np.ndarray, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Copies `packed` to the device: into this ring entry's own device
        buffer, or into `into` (a buffer whose address a captured graph reads)."""
        i = self.turn
        self.turn = (self.turn + 1) % self.depth
        n = packed.shape[0]
        if self.host[i] is None or self.host[i].numel() < n:
            cap = max(1024, 1 << (n - 1).bit_length())
            self.host[i] = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self.dev[i] = torch.empty(cap, dtype=torch.int32, device=self.device)
        if self.events[i] is not None:
            self.events[i].synchronize()     # the copy that last read this host buffer has run
        self.host[i][:n].numpy()[:] = packed
        target = self.dev[i] if into is None else into
        target[:n].copy_(self.host[i][:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev
        return target


class _DecodeGraph:
    """A captured decode step for one batch shape: `rows` single-token requests
    whose block tables are `table_width` pages wide. Its index arrays, its
    scratch and its logits live at fixed addresses; a replay reads new indices
    from the same place."""

    def __init__(self):
        self.graph = None
        self.meta: Optional[torch.Tensor] = None
        self.workspace: Optional[Workspace] = None
        self.logits: Optional[torch.Tensor] = None
        self.seen = 0


TABLE_BUCKET = 8     # captured steps round their block-table width up to this many pages


class Engine:
    def __init__(self, model_dir: str, dtype: str = "bfloat16", max_tokens: int = 8192, page_size: int = 64,
                 max_requests: int = 64, device: str = "cuda:0", use_graphs: bool = True):
        if dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        library()                       # fail now, and loudly, if the kernels are missing
        if not torch.cuda.is_available():
            raise RuntimeError("imparo_amd runs on a GPU; none is visible to this process")
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.dtype = DTYPES[dtype]
        self.model_dir = model_dir
        self.config_json = read_config_json(model_dir)
        self.config, self.plan = plan_from_config(self.config_json)
        declared = declared_tensors(self.plan)
        tensors = load_weights(model_dir, {k: d for k, (d, _) in declared.items()})
        self.model = Model(self.plan, tensors, self.device, self.dtype)
        f = tensors.pop("__file__", None)
        del tensors
        if f is not None:
            f.close()
        self.page_size = page_size
        n_pages = max(1, math.ceil(max_tokens / page_size))
        self.cache = CacheManager(self.model.site_specs, page_size, n_pages, max_requests)
        self.storage = CacheStorage(self.cache, self.dtype, self.device)
        self.workspace = Workspace(self.device)
        self._upload = _Upload(self.device)
        # decode steps (every request brings one token and wants its logits) replay a captured
        # HIP graph: the launches of a step cost more host time than the step's kernels take
        self.use_graphs = use_graphs
        self._graphs: Dict[Tuple[int, int], _DecodeGraph] = {}
        self._graph_pool = None
        self.vocab_size = self.plan.vocab_size
        self.max_position = self.plan.max_position
        self.steps_run = 0

    # ------------------------------------------------------------ requests
    def length(self, request: Hashable) -> int:
        return self.cache.length.get(request, 0)

    def is_live(self, request: Hashable) -> bool:
        return self.cache.is_live(request)

    def release(self, request: Hashable) -> None:
        """The request is finished: its pages and its slot are given back."""
        if self.cache.is_live(request):
            self.cache.release(request)

    def free_pages(self) -> List[int]:
        return self.cache.free_pages()

    # ------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Runs one batch. Returns float32 logits [wanted, vocab] on the
        device, in the order of the entries and of each entry's `want`, or
        None when nothing is wanted."""
        entries = [e for e in entries]
        seen = set()
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if len(e.tokens) == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            for tok in e.tokens:
                if not 0 <= int(tok) < self.vocab_size:
                    raise StepError(f"request {e.request!r}: token id {tok} is outside the vocabulary "
                                    f"of {self.vocab_size}")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise StepError(f"request {e.request!r}: wanted place {w} is outside its "
                                    f"{len(e.tokens)} tokens")
            if self.length(e.request) + len(e.tokens) > self.max_position:
                raise StepError(f"request {e.request!r} would pass the model's {self.max_position} positions")
        if not entries:
            return None

        # pages and slots, all or nothing
        admitted: List[Hashable] = []
        taken: List[Tuple[Hashable, list]] = []
        try:
            for e in entries:
                if not self.cache.is_live(e.request):
                    slot = self.cache.admit(e.request)
                    admitted.append(e.request)
                    self.storage.zero_slot(slot)
                got = self.cache.reserve(e.request, self.cache.length[e.request] + len(e.tokens))
                taken.append((e.request, got))
        except OutOfPages:
            for req, got in reversed(taken):
                self.cache.rollback(req, got)
            for req in admitted:
                self.cache.release(req)
            raise

        if (self.use_graphs and self.model.graph_safe
                and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)):
            logits = self._decode_step(entries)
        else:
            ctx, token_ids, want_rows = self._pack(entries)
            logits = self.model.forward(ctx, token_ids, want_rows)
        for e in entries:
            self.cache.commit(e.request, self.cache.length[e.request] + len(e.tokens))
        self.steps_run += 1
        return logits

    def _decode_step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """A step of single tokens. The first step of a batch shape runs
        launch by launch (so that every kernel it needs has been loaded), the
        second is captured, later ones replay the capture."""
        G = len(self.cache.groups)
        widest = max([self.cache.table_len(g, e.request) for e in entries for g in range(G)] or [1])
        width = -(-widest // TABLE_BUCKET) * TABLE_BUCKET
        key = (len(entries), width)
        g = self._graphs.setdefault(key, _DecodeGraph())
        g.seen += 1
        if g.seen == 1:
            ctx, token_ids, want_rows = self._pack(entries)
            return self.model.forward(ctx, token_ids, want_rows)
        if g.graph is None:
            g.workspace = Workspace(self.device)
            # the capture fixes grid sizes: they are sized for the widest context the tables can hold
            ctx, token_ids, want_rows = self._pack(entries, table_width=width, workspace=g.workspace, graph=g)
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                g.logits = self.model.forward(ctx, token_ids, want_rows)
            g.graph = graph
        else:
            self._pack(entries, table_width=width, workspace=g.workspace, graph=g)
        g.graph.replay()
        return g.logits

    def _pack(self, entries: Sequence[StepEntry], table_width: Optional[int] = None,
              workspace: Optional[Workspace] = None, graph: Optional[_DecodeGraph] = None):
        """Builds the step's index arrays, sends them to the device in one
        copy and wraps them in a StepContext. For a captured step the arrays go
        to the capture's own fixed buffer and sizes are the capture's bounds."""
        a, lay = self.cache.pack([e.request for e in entries], [e.tokens for e in entries],
                                 [e.want for e in entries], table_width or 0)
        T, R, W, G, P, total = lay["T"], lay["R"], lay["W"], lay["G"], lay["P"], lay["total"]
        o_pos, o_row = T, 2 * T
        o_start, o_len, o_slot = 3 * T, 3 * T + R, 3 * T + 2 * R
        o_lists = 3 * T + 3 * R
        o_want = 3 * T + 4 * R
        o_tab = o_want + W
        o_tok = 0
        n_dec = lay["n_single"]
        if graph is not None:
            if graph.meta is None:
                graph.meta = torch.empty(total, dtype=torch.int32, device=self.device)
            dev = self._upload.send(a, into=graph.meta)
        else:
            dev = self._upload.send(a)
        block_tables = {g: dev[o_tab + g * R * P:o_tab + (g + 1) * R * P].view(R, P) for g in range(G)}
        ctx = StepContext(
            n_tokens=T, n_rows=R,
            positions=dev[o_pos:o_pos + T], row_of_token=dev[o_row:o_row + T],
            seg_start=dev[o_start:o_start + R], seg_len=dev[o_len:o_len + R], slot=dev[o_slot:o_slot + R],
            block_tables=block_tables, page_size=self.page_size, dtype=self.dtype,
            workspace=workspace or self.workspace, storage=self.storage, group_of_site=self.cache.group_of_site,
            max_seg_len=lay["max_seg_len"],
            max_context=lay["max_context"] if table_width is None else table_width * self.page_size,
            decode_rows=dev[o_lists:o_lists + n_dec], n_decode_rows=n_dec,
            prefill_rows=dev[o_lists + n_dec:o_lists + R], n_prefill_rows=lay["n_multi"],
            n_prefill_tiles=lay["n_prefill_tiles"],
        )
        want_rows = dev[o_want:o_want + W] if W else None
        return ctx, dev[o_tok:o_tok + T], want_rows
