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
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pages import CacheError, CacheManager
from ..cache.storage import CacheStorage
from ..config import plan_from_config, read_config_json
from ..kernels import library, ops
from ..kernels.program import StepArgs
from ..parts.base import StepContext, Workspace
from ..weights import load_weights
from .model import Model, declared_tensors

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


class StepError(ValueError):
    """A batch the step function refuses; nothing has changed."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]          # token ids; a lone DeviceToken stands for one that was not read back yet
    want: Sequence[int] = ()       # places among `tokens` whose logits are wanted


@dataclass(frozen=True)
class DeviceToken:
    """A token id that the sampling kernel left on the device: element `index`
    of `source`, an int32 tensor. A request may bring one as its only token;
    the step then takes the id from there, so that the host need not wait for
    the step before to end before it queues the next."""
    source: torch.Tensor
    index: int


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
    whose block tables are `table_width` pages wide. Its index arrays live at an
    address of its own; scratch and logits are the engine's (buffers never move,
    and the capture keeps those it was recorded with alive)."""

    def __init__(self):
        self.graph = None
        self.meta: Optional[torch.Tensor] = None
        self.pinned: list = []
        self.logits: Optional[torch.Tensor] = None
        self.last_used = 0


REGION_CAP = 256 << 20   # bytes of one scratch region that are reserved up front; beyond that it grows when needed
TABLE_BUCKET = 8     # captured steps round their block-table width up to a multiple of this many pages, or more
MAX_GRAPHS = 256     # captured batch shapes kept (more if `warm` is asked for more); beyond that the one unused for longest goes


def table_bucket(pages: int) -> int:
    """The block-table width a captured step is sized for: `pages` rounded up to a multiple of 8 up to 127
    pages, of 16 up to 255, of 32 up to 511, and so on: at most an eighth wider than the longest context
    needs (the attention grid is sized by it, and a split nobody needs still costs its blocks' launch:
    0.7 us a layer for each 256 keys too many at 13 rows), and a long run meets few widths (a shape is a
    number of rows and a width, and a new one costs several steps' time to capture)."""
    step = TABLE_BUCKET
    while step * 16 <= pages:
        step *= 2
    return -(-pages // step) * step


class Engine:
    """`max_tokens`: the most tokens that live requests hold at any time, each
    request's count rounded up to whole pages; the pools are made for that
    many. Instead, `kv_budget_bytes` gives the memory the paged caches may
    take and the pools are as large as fits (the reference sizes its pool
    from a memory budget the same way and carries a cap in pages for tests,
    /root/reference/crates/imparo-model/src/kv.rs:574-621), or `num_pages`
    gives the pool size outright (one number, or one per cache group).
    `max_step_tokens` bounds the tokens of one step; a larger batch is refused.
    `native_step`: a step's kernels are issued by one call into the kernel
    library (a step program) where every part of the model can describe itself
    to it; False, or a model with a part that cannot, runs the parts one by one
    from here. Both issue the same kernels with the same arguments, except that
    the native step may fold a norm into the products around it in steps of at
    most 16 single tokens (`fold_norms`: None where the library's plan says it
    pays, False never, True wherever possible), which changes results by
    rounding only."""

    def __init__(self, model_dir: str, dtype: str = "bfloat16", max_tokens: Optional[int] = None, page_size: int = 64,
                 max_requests: int = 64, device: str = "cuda:0", use_graphs: bool = True,
                 kv_budget_bytes: Optional[int] = None, num_pages=None, max_step_tokens: int = 8192,
                 native_step: bool = True, fold_norms: Optional[bool] = None):
        if dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        if sum(x is not None for x in (max_tokens, kv_budget_bytes, num_pages)) > 1:
            raise ValueError("give one of max_tokens, kv_budget_bytes and num_pages")
        if max_step_tokens < 1:
            raise ValueError(f"max_step_tokens must be at least 1, got {max_step_tokens}")
        library()                       # fail now, and loudly, if the kernels are missing
        if not torch.cuda.is_available():
            raise RuntimeError("imparo_amd runs on a GPU; none is visible to this process")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise ValueError(f"imparo_amd runs on a GPU; {device!r} is none")
        if self.device.index is None:       # "cuda" means the current one; tensors report an index
            self.device = torch.device("cuda", torch.cuda.current_device())
        torch.cuda.set_device(self.device)
        self.dtype = DTYPES[dtype]
        self.model_dir = model_dir
        self.config_json = read_config_json(model_dir)
        self.config, self.plan = plan_from_config(self.config_json)
        declared = declared_tensors(self.plan)
        tensors = load_weights(model_dir, {k: d for k, (d, _) in declared.items()}, self.plan.restated_tensors)
        self.model = Model(self.plan, tensors, self.device, self.dtype, page_size)
        f = tensors.pop("__file__", None)
        del tensors
        if f is not None:
            f.close()
        self.page_size = page_size
        self.max_step_tokens = max_step_tokens
        pool_sizes = self.pool_sizes(self.model.site_specs, page_size, self.dtype, max_tokens, kv_budget_bytes,
                                     num_pages)
        self.cache = CacheManager(self.model.site_specs, page_size, pool_sizes, max_requests)
        self.storage = CacheStorage(self.cache, self.dtype, self.device)
        self.workspace = Workspace(self.device)
        self._upload = _Upload(self.device)
        # decode steps (every request brings one token and wants its logits) replay a captured
        # HIP graph: the launches of a step cost more host time than the step's kernels take
        self.use_graphs = use_graphs
        self._graphs: Dict[Tuple[int, int], _DecodeGraph] = {}
        self.max_graphs = MAX_GRAPHS
        self._graph_pool = None
        self._capture_stream = None
        self.vocab_size = self.plan.vocab_size
        self.max_position = self.plan.max_position
        self.steps_run = 0
        ops.load_code()                 # every kernel file's code is on the device before any capture
        self.program = (self.model.build_program(self.storage, self.cache.group_of_site, page_size)
                        if native_step else None)
        self._args = StepArgs()
        self._prefill_tile = ops.prefill_tile()
        if self.program is not None:
            self.program.set_fold(1 if fold_norms is None else (2 if fold_norms else 0))
            self._size_workspace(max_requests)

    @staticmethod
    def pool_sizes(site_specs, page_size: int, dtype: torch.dtype, max_tokens: Optional[int],
                   kv_budget_bytes: Optional[int], num_pages) -> List[int]:
        """Pages per cache group. From `num_pages` as given; from a budget in
        bytes: every group the same number of pages, as many as the budget
        pays for over all sites (a page of a group costs page_size x the bytes
        its sites keep per position); else from `max_tokens` (default 8,192)."""
        groups = CacheManager.groups_of(site_specs)
        if num_pages is not None:
            sizes = [int(num_pages)] * len(groups) if isinstance(num_pages, int) else [int(n) for n in num_pages]
            if len(sizes) != len(groups) or any(n < 1 for n in sizes):
                raise ValueError(f"num_pages {num_pages!r} does not give {len(groups)} cache groups a pool each")
            return sizes
        if kv_budget_bytes is not None:
            element = 4 if dtype == torch.float32 else 2
            per_page = sum(spec.bytes_per_position(element) * len(sites) * page_size for spec, sites in groups)
            if per_page == 0:
                return []
            n = int(kv_budget_bytes) // per_page
            if n < 1:
                raise ValueError(f"a cache budget of {kv_budget_bytes} bytes does not pay for one page of "
                                 f"{per_page} bytes over all sites")
            return [n] * len(groups)
        tokens = 8192 if max_tokens is None else max_tokens
        return [max(1, math.ceil(tokens / page_size))] * len(groups)

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
        None when nothing is wanted. The tensor is the engine's: a later step
        may write its own logits there, so use it (or copy it) before the next.
        A batch that is refused (StepError) changes nothing. A step that fails
        once its kernels have started leaves no request of the batch live."""
        entries = list(entries)
        if not entries:
            return None
        n_tokens = sum(len(e.tokens) for e in entries)
        if n_tokens > self.max_step_tokens:
            raise StepError(f"a step of {n_tokens} tokens passes this engine's bound of {self.max_step_tokens} "
                            f"(max_step_tokens); cut the prompts into smaller portions")
        # the native side checks the batch, admits, and reserves pages and slots, all or nothing
        token_lists = [e.tokens for e in entries]
        on_device = [(row, e.tokens[0]) for row, e in enumerate(entries)
                     if len(e.tokens) == 1 and isinstance(e.tokens[0], DeviceToken)]
        for row, tok in on_device:
            if (tok.source.dtype != torch.int32 or tok.source.dim() != 1 or tok.source.device != self.device
                    or not 0 <= tok.index < tok.source.shape[0] or tok.source is not on_device[0][1].source):
                raise StepError(f"request {entries[row].request!r}: a device token must be an element of one "
                                f"int32 vector on {self.device}, the same for the whole step")
            token_lists[row] = (0,)          # a placeholder until the id is copied in on the device
        try:
            batch = self.cache.batch([e.request for e in entries], token_lists, [e.want for e in entries])
        except CacheError as err:
            raise StepError(str(err)) from None
        if on_device:
            starts = np.cumsum(batch.n_tok) - batch.n_tok
            batch.device_tokens = (on_device[0][1].source,
                                   np.array([starts[row] for row, _ in on_device], dtype=np.int32),
                                   np.array([tok.index for _, tok in on_device], dtype=np.int32))
        code, row = self.cache.begin_step(batch, self.vocab_size, self.max_position)
        if code:
            raise StepError(self._refusal(code, entries[row]))
        try:
            with ops.on_current_stream():
                for slot in batch.new_slots[batch.new_slots >= 0].tolist():
                    self.storage.reset_slot(slot)
            if (self.use_graphs and self.model.graph_safe and batch.T == len(entries)
                    and bool((batch.n_want == 1).all())):
                logits = self._decode_step(entries, batch)       # one token each, wanted
            else:
                logits = self._run(self._pack(batch))
        except BaseException:
            # Pages and new admissions are rolled back. Fixed-size state is not a thing that can be
            # rolled back (a conv history has been shifted by the layers that ran), so the requests
            # of a step that failed after its first launch cannot go on: they are released, and a
            # caller that wants them recomputes them from their tokens.
            self.cache.abort_step(batch)
            for e in entries:
                self.release(e.request)
            raise
        self.cache.end_step(batch)
        self.steps_run += 1
        return logits

    def _refusal(self, code: int, e: StepEntry) -> str:
        from ..cache import native as N
        if code == N.E_TWICE:
            return f"request {e.request!r} appears twice in one step"
        if code == N.E_EMPTY:
            return f"request {e.request!r} brings no tokens"
        if code == N.E_POSITIONS:
            return f"request {e.request!r} would pass the model's {self.max_position} positions"
        if code == N.E_TOKEN:
            bad = next(t for t in e.tokens if not 0 <= int(t) < self.vocab_size)
            return f"request {e.request!r}: token id {bad} is outside the vocabulary of {self.vocab_size}"
        if code == N.E_WANT:
            bad = next(w for w in e.want if not 0 <= int(w) < len(e.tokens))
            return f"request {e.request!r}: wanted place {bad} is outside its {len(e.tokens)} tokens"
        return f"request {e.request!r}: the cache manager refused the step with code {code}"

    def _decode_step(self, entries: Sequence[StepEntry], batch) -> torch.Tensor:
        """A step of single tokens: a batch shape is captured when it first
        comes and replayed from then on."""
        width = table_bucket(batch.widest)
        g = self._graph_for(len(entries), width)
        if g.graph is None:
            self._capture(g, self._pack(batch, table_width=width, graph=g))
        else:
            self._pack(batch, table_width=width, graph=g)
        g.graph.replay()
        return g.logits

    def _graph_for(self, rows: int, width: int) -> _DecodeGraph:
        key = (rows, width)
        g = self._graphs.get(key)
        if g is None:
            if len(self._graphs) >= self.max_graphs:      # each holds an executable graph and its index arrays
                del self._graphs[min(self._graphs, key=lambda k: self._graphs[k].last_used)]
            g = self._graphs[key] = _DecodeGraph()
        g.last_used = self.steps_run
        return g

    def _capture(self, g: _DecodeGraph, packed: "_Packed") -> None:
        """Records the step that `packed` describes into `g`. The capture fixes grid sizes: they are
        sized for the widest context the tables can hold."""
        if self.program is not None:
            self._grow_for(packed)                   # a capture must not meet a region that is too small
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        # Captured by hand, on a stream of its own: the library's context manager waits for the device, collects
        # garbage and empties the allocator's cache before every capture, which is most of what a new shape costs.
        if self._capture_stream is None:
            self._capture_stream = torch.cuda.Stream(device=self.device)
        here = torch.cuda.current_stream(self.device)
        self._capture_stream.wait_stream(here)
        with torch.cuda.stream(self._capture_stream):
            graph.capture_begin(pool=self._graph_pool)
            try:
                g.logits = self._run(packed)
            finally:
                graph.capture_end()
        here.wait_stream(self._capture_stream)
        g.pinned = self.workspace.pin()          # the buffers whose addresses the graph holds
        g.graph = graph

    def warm(self, rows: Sequence[int], contexts: Sequence[int] = (1,)) -> int:
        """Captures the decode steps of `rows` single-token requests whose longest context is
        `contexts` tokens, for every pair of the two, before any request needs them: a shape that is
        met for the first time while serving costs several steps' time. Returns how many shapes it
        captured. Nothing runs and no request is touched: a capture records launches only."""
        made = 0
        if not (self.use_graphs and self.model.graph_safe):
            return made
        G = len(self.cache.groups)
        rows, contexts = sorted(set(int(r) for r in rows)), sorted(set(int(c) for c in contexts))
        if any(n < 1 for n in rows) or any(c < 1 for c in contexts):
            raise ValueError("warm: rows and contexts are positive numbers")
        wanted = {(n, table_bucket(-(-c // self.page_size))) for n in rows for c in contexts}
        # what the caller asks for is kept: room for all of it beside what is there
        self.max_graphs = max(self.max_graphs, len(set(self._graphs) | wanted))
        for n in rows:
            for context in contexts:
                width = table_bucket(-(-context // self.page_size))
                g = self._graph_for(n, width)
                if g.graph is not None:
                    continue
                lay = dict(T=n, R=n, W=n, G=G, P=width, n_single=n, n_multi=0, max_seg_len=1,
                           max_context=width * self.page_size, total=3 * n + 4 * n + n + G * n * width)
                g.meta = torch.zeros(lay["total"] + 2 * n, dtype=torch.int32, device=self.device)
                self._capture(g, _Packed(g.meta, lay, width * self.page_size, np.ones(n, dtype=np.int32)))
                made += 1
        return made

    def _pack(self, batch, table_width: Optional[int] = None, graph: Optional[_DecodeGraph] = None) -> "_Packed":
        """Builds the step's index arrays and sends them to the device in one
        copy. For a captured step the arrays go to the capture's own fixed
        buffer and sizes are the capture's bounds."""
        a, lay = self.cache.pack_batch(batch, table_width or 0)
        T, R, total = lay["T"], lay["R"], lay["total"]
        placed = batch.device_tokens
        if placed is not None:               # where the ids go, and where they come from, ride along
            a = np.concatenate([a, placed[1], placed[2]])
        if graph is not None:
            if graph.meta is None:
                graph.meta = torch.empty(total + 2 * R, dtype=torch.int32, device=self.device)
            dev = self._upload.send(a, into=graph.meta)
        else:
            dev = self._upload.send(a)
        if placed is not None:
            n = placed[1].shape[0]
            with ops.on_current_stream():
                ops.place_tokens(dev[:T], dev[total:total + n], placed[0], dev[total + n:total + 2 * n], self.vocab_size)
        return _Packed(dev, lay, lay["max_context"] if table_width is None else table_width * self.page_size,
                       batch.n_tok)

    def _run(self, packed: "_Packed") -> Optional[torch.Tensor]:
        """Issues the kernels of a packed step on the current stream and returns its logits."""
        if self.program is None:
            ctx, token_ids, want_rows = self._context(packed)
            with ops.on_current_stream():
                return self.model.forward(ctx, token_ids, want_rows)
        W = packed.lay["W"]
        at = self.program.run(self._step_args(packed), self.workspace, torch.cuda.current_stream().cuda_stream)
        if at is None:
            return None
        logits = self.workspace.get("logits", (W, self.vocab_size), torch.float32)
        assert logits.data_ptr() == at
        return logits

    def _step_args(self, packed: "_Packed") -> StepArgs:
        """The packed step as the native program takes it: addresses inside the one device array."""
        lay = packed.lay
        T, R, W, G, P = lay["T"], lay["R"], lay["W"], lay["G"], lay["P"]
        base = packed.dev.data_ptr()
        n_single = lay["n_single"]
        at = lambda offset: base + 4 * offset
        a = self._args
        a.tokens, a.positions, a.row_of_token = at(0), at(T), at(2 * T)
        a.seg_start, a.seg_len, a.slot = at(3 * T), at(3 * T + R), at(3 * T + 2 * R)
        a.single_rows, a.portion_rows = at(3 * T + 3 * R), at(3 * T + 3 * R + n_single)
        a.want_rows = at(3 * T + 4 * R)
        tables = 3 * T + 4 * R + W
        if G > len(a.tables):
            raise StepError(f"the step program takes {len(a.tables)} cache groups, this model has {G}")
        for g in range(G):
            a.tables[g] = at(tables + g * R * P)
        a.n_groups, a.table_width = G, P
        a.n_tokens, a.n_rows, a.n_want, a.n_single, a.n_portion = T, R, W, n_single, lay["n_multi"]
        a.max_seg_len, a.max_context = lay["max_seg_len"], packed.max_context
        n = packed.host_seg_len
        tile = self._prefill_tile
        a.portion_tiles = int(((n[n > 1] + (tile - 1)) // tile).sum()) if lay["n_multi"] else 0
        return a

    def _step_args_for_rows(self, rows: int, context: Optional[int] = None) -> StepArgs:
        """The shape of a step of `rows` single tokens (no addresses): for asking the program what such a step uses."""
        a = self._args
        context = context or self.page_size
        a.n_groups, a.table_width = len(self.cache.groups), -(-context // self.page_size)
        a.n_tokens, a.n_rows, a.n_want, a.n_single, a.n_portion = rows, rows, rows, rows, 0
        a.max_seg_len, a.max_context, a.portion_tiles = 1, context, 0
        return a

    def _grow_for(self, packed: "_Packed") -> None:
        for name, need in self.program.needs(self._step_args(packed)).items():
            self.workspace.reserve(name, need)

    def _size_workspace(self, max_requests: int) -> None:
        """Reserves the program's scratch for the largest steps this engine takes, so that no step
        meets a buffer that must grow: steps of 1 to `max_requests` single tokens, and steps of one
        portion of up to `max_step_tokens` tokens, each at the longest context the pools can hold.
        A region that would pass REGION_CAP is left to grow when a step needs it (the partial
        results of very long contexts)."""
        G = len(self.cache.groups)
        longest = max([self.page_size] + [g.pool.n_pages * self.page_size for g in self.cache.groups])
        longest = min(longest, self.max_position)
        a = self._args
        need: Dict[str, int] = {}

        def shape(T, R, single, context):
            a.n_groups, a.table_width = G, -(-context // self.page_size)
            a.n_tokens, a.n_rows, a.n_want = T, R, R
            a.n_single, a.n_portion = (R, 0) if single else (0, R)
            a.max_seg_len, a.max_context = (1 if single else T), context
            a.portion_tiles = 0 if single else -(-T // self._prefill_tile)
            for name, n in self.program.needs(a).items():
                need[name] = max(need.get(name, 0), n)

        for rows in range(1, max_requests + 1):
            shape(rows, rows, True, longest)
        # (the products' slices of K depend on the rows: every count to 64, then every 16th to 512, then doublings)
        sizes = {n for n in list(range(2, 65)) + list(range(80, 513, 16)) if n <= self.max_step_tokens}
        sizes |= {n for n in (1024, 2048, 4096, 8192, 16384) if n < self.max_step_tokens} | {self.max_step_tokens}
        for tokens in sorted(sizes):
            shape(tokens, 1, False, min(longest, max(tokens, self.page_size)))
            shape(tokens, 1, False, longest)
        for name, n in need.items():
            self.workspace.reserve(name, min(n, REGION_CAP))
        self.program.bind(self.workspace)

    def _context(self, packed: "_Packed"):
        """The packed step as the parts see it when they run one by one."""
        dev, lay = packed.dev, packed.lay
        T, R, W, G, P = lay["T"], lay["R"], lay["W"], lay["G"], lay["P"]
        o_pos, o_row = T, 2 * T
        o_start, o_len, o_slot = 3 * T, 3 * T + R, 3 * T + 2 * R
        o_lists = 3 * T + 3 * R
        o_want = 3 * T + 4 * R
        o_tab = o_want + W
        n_dec = lay["n_single"]
        block_tables = {g: dev[o_tab + g * R * P:o_tab + (g + 1) * R * P].view(R, P) for g in range(G)}
        ctx = StepContext(
            n_tokens=T, n_rows=R,
            positions=dev[o_pos:o_pos + T], row_of_token=dev[o_row:o_row + T],
            seg_start=dev[o_start:o_start + R], seg_len=dev[o_len:o_len + R], slot=dev[o_slot:o_slot + R],
            block_tables=block_tables, page_size=self.page_size, dtype=self.dtype,
            workspace=self.workspace, storage=self.storage, group_of_site=self.cache.group_of_site,
            max_seg_len=lay["max_seg_len"], max_context=packed.max_context,
            single_rows=dev[o_lists:o_lists + n_dec], n_single_rows=n_dec,
            portion_rows=dev[o_lists + n_dec:o_lists + R], n_portion_rows=lay["n_multi"],
            host_seg_len=packed.host_seg_len,
        )
        want_rows = dev[o_want:o_want + W] if W else None
        return ctx, dev[:T], want_rows


class _Packed:
    """A step's index arrays on the device (one int32 array, laid out as the cache manager packs
    them), the sizes of its parts, the bound on every row's context, tokens per row on the host."""
    __slots__ = ("dev", "lay", "max_context", "host_seg_len")

    def __init__(self, dev: torch.Tensor, lay: Dict[str, int], max_context: int, host_seg_len):
        self.dev, self.lay, self.max_context, self.host_seg_len = dev, lay, max_context, host_seg_len
