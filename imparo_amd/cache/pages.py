"""Host-side bookkeeping of the cache: pages, block tables, state slots.

The bookkeeping itself is native (csrc/host/cache_manager.cpp, reached through
a C ABI); the classes here give it Python names and errors. Nothing here
touches the GPU; the tensors the pages index live in
`imparo_amd.cache.storage`.

Allocation always takes the lowest free page, so which pages a request gets
is a function of which pages are free and never of history; freeing a page
twice is an error. The reference's block allocator keeps the same two rules
(/root/reference/crates/imparo-kv/src/alloc.rs:1-11,51-75).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from itertools import chain
from typing import Dict, Hashable, Iterator, List, Optional, Sequence, Tuple, Union

import numpy as np

from . import native as N


class OutOfPages(RuntimeError):
    """The pool cannot give the pages (or the slot) a step needs."""


class CacheError(RuntimeError):
    """Misuse of the cache manager: a page freed twice, an unknown request."""


class PagePool:
    """A pool of pages: the lowest free page first, always."""

    def __init__(self, n_pages: int, _borrowed=None):
        self._lib = N.host_library()
        if _borrowed is not None:
            self._p, self._owned = _borrowed, False
        else:
            if n_pages < 0:
                raise ValueError("a pool cannot have a negative number of pages")
            self._p, self._owned = self._lib.imparo_pool_new(n_pages), True

    def __del__(self):
        if getattr(self, "_owned", False) and self._p:
            self._lib.imparo_pool_delete(self._p)
            self._p = None

    @property
    def n_pages(self) -> int:
        return self._lib.imparo_pool_n_pages(self._p)

    @property
    def n_free(self) -> int:
        return self._lib.imparo_pool_n_free(self._p)

    @property
    def high_water(self) -> int:
        """One past the highest page ever handed out."""
        return self._lib.imparo_pool_high_water(self._p)

    def alloc(self) -> int:
        page = self._lib.imparo_pool_alloc(self._p)
        if page < 0:
            raise OutOfPages("no free page")
        return page

    def free(self, page: int) -> None:
        rc = self._lib.imparo_pool_free(self._p, page)
        if rc == N.E_RANGE:
            raise CacheError(f"page {page} is outside the pool of {self.n_pages}")
        if rc == N.E_DOUBLE_FREE:
            raise CacheError(f"page {page} freed twice")

    def is_free(self, page: int) -> bool:
        return self._lib.imparo_pool_is_free(self._p, page) == 1

    def scramble(self, seed: int) -> None:
        """Permutes which physical page each allocation rank maps to, so that
        block tables are not the identity. Only on an untouched pool. Output
        must not depend on it: placement is invisible
        (/root/reference/crates/imparo-kv/src/resident.rs:56-99)."""
        if self._lib.imparo_pool_scramble(self._p, seed) != 0:
            raise CacheError("placement can only be scrambled while every page is free")


PAGE = -1     # in a PagedArray's page shape: the dimension that runs over the positions of a page


@dataclass(frozen=True)
class PagedArray:
    """One tensor of a paged cache site: the shape of one page of it, with
    PAGE where the page's positions run, and whether it is kept in float32
    instead of the engine's dtype. The device tensor is [n_pages, *page_shape]."""
    name: str
    page_shape: Tuple[int, ...]
    float32: bool = False

    def shape(self, n_pages: int, page_size: int) -> Tuple[int, ...]:
        return (n_pages,) + tuple(page_size if d == PAGE else d for d in self.page_shape)

    def elements_per_position(self) -> int:
        n = 1
        for d in self.page_shape:
            n *= 1 if d == PAGE else d
        return n


@dataclass(frozen=True)
class PagedSpec:
    """State that grows with the context, in pages: the arrays a mixer keeps
    per position (keys and values, a latent, whatever it declares), laid out
    as the mixer's kernels read them. `window` None keeps every position; a
    number keeps only that many. Sites with equal specs share a pool and a
    block table per request."""
    arrays: Tuple[PagedArray, ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [a.name for a in self.arrays]
        if len(set(names)) != len(names):
            raise ValueError(f"a paged spec names an array twice: {names}")
        for a in self.arrays:
            if list(a.page_shape).count(PAGE) != 1:
                raise ValueError(f"array {a.name!r}: exactly one dimension of a page's shape runs over its positions")

    def bytes_per_position(self, element_size: int) -> int:
        return sum(a.elements_per_position() * (4 if a.float32 else element_size) for a in self.arrays)


def kv_spec(kv_heads: int, head_dim: int, window: Optional[int] = None, v_transposed: bool = False) -> PagedSpec:
    """Keys and values of grouped-query attention: K [kv_heads, page, head_dim]
    and V the same, or transposed inside the page [kv_heads, head_dim, page]."""
    v_shape = (kv_heads, head_dim, PAGE) if v_transposed else (kv_heads, PAGE, head_dim)
    return PagedSpec((PagedArray("k", (kv_heads, PAGE, head_dim)), PagedArray("v", v_shape)), window)


@dataclass(frozen=True)
class FixedArray:
    """One tensor of a fixed-size state: its shape per request, its dtype
    ("float32", "bfloat16", "int32", or "engine" for the engine's own dtype)
    and the value a request that has seen nothing starts from (anything but
    float32 starts from zero). The device tensor is [n_slots, *shape]."""
    name: str
    shape: Tuple[int, ...]
    dtype: str = "float32"
    init: float = 0.0

    def __post_init__(self):
        if self.dtype not in ("float32", "bfloat16", "int32", "engine"):
            raise ValueError(f"state array {self.name!r}: dtype {self.dtype!r} is none of float32, bfloat16, int32, engine")
        if self.dtype != "float32" and self.init != 0.0:
            raise ValueError(f"state array {self.name!r}: only a float32 array can start from a value other than zero")


@dataclass(frozen=True)
class FixedSpec:
    """State of a fixed size per request (a conv history, a recurrent matrix).
    `FixedSpec(shape, init)` is one float32 array, named "state"; a mixer that
    keeps several tensors of different shapes or dtypes (a recurrent matrix
    beside a short history, a 16-bit state) names them in `arrays` instead."""
    shape: Optional[Tuple[int, ...]] = None
    init: float = 0.0
    arrays: Tuple[FixedArray, ...] = ()

    def __post_init__(self):
        if (self.shape is None) == (len(self.arrays) == 0):
            raise ValueError("a fixed spec is either one float32 array (shape, init) or a tuple of named arrays")
        names = [a.name for a in self.arrays]
        if len(set(names)) != len(names):
            raise ValueError(f"a fixed spec names an array twice: {names}")

    def all_arrays(self) -> Tuple[FixedArray, ...]:
        return self.arrays or (FixedArray("state", tuple(self.shape), "float32", self.init),)


StateSpec = Union[PagedSpec, FixedSpec, None]


class _Tables:
    """The block tables of one group, by request: a read-only mapping."""

    def __init__(self, manager: "CacheManager", group: int):
        self._m, self._g = manager, group

    def __getitem__(self, req: Hashable) -> List[int]:
        return self._m.table(self._g, req)

    def __iter__(self) -> Iterator[Hashable]:
        return iter(self._m._live_names())

    def __len__(self) -> int:
        return len(self._m._live_names())

    def __contains__(self, req: Hashable) -> bool:
        return self._m.is_live(req)

    def keys(self):
        return self._m._live_names()

    def values(self):
        return [self[r] for r in self.keys()]

    def items(self):
        return [(r, self[r]) for r in self.keys()]


class CacheGroup:
    """The cache sites that share one paged spec: one pool of pages, one block
    table per request, the same page ids on every site of the group."""

    def __init__(self, manager: "CacheManager", index: int, spec: PagedSpec, pool: PagePool, page_size: int):
        self._m, self.index = manager, index
        self.spec = spec
        self.sites: List[int] = []
        self.page_size = page_size
        self.pool = pool
        self.tables = _Tables(manager, index)

    def first_needed_page(self, next_position: int) -> int:
        """The lowest logical page a query at `next_position` or later reads."""
        return self._m._lib.imparo_cache_first_needed_page(self._m._c, self.index, next_position)


class _PerRequest:
    """cache.length / cache.slot_of: read-only mappings over the live requests."""

    def __init__(self, manager: "CacheManager", fn):
        self._m, self._fn = manager, fn

    def __getitem__(self, req: Hashable) -> int:
        if not self._m.is_live(req):
            raise KeyError(req)
        return self._fn(self._m._c, self._m._handles[req])

    def get(self, req: Hashable, default=None):
        return self[req] if self._m.is_live(req) else default

    def __contains__(self, req: Hashable) -> bool:
        return self._m.is_live(req)

    def __iter__(self):
        return iter(self._m._live_names())

    def values(self):
        return [self[r] for r in self._m._live_names()]

    def items(self):
        return [(r, self[r]) for r in self._m._live_names()]


class CacheManager:
    """Pages and slots of every live request.

    A request is admitted (gets a state slot, empty tables), grows by
    `reserve` (pages for the positions a step will write) followed by
    `commit` (the step ran) or `rollback` (it did not), and leaves by
    `release`, which gives back everything it holds.
    """

    @staticmethod
    def groups_of(site_specs: Sequence[StateSpec]) -> List[Tuple[PagedSpec, List[int]]]:
        """The groups a list of site specs makes: (spec, its sites), in order of first appearance."""
        out: List[Tuple[PagedSpec, List[int]]] = []
        for site, spec in enumerate(site_specs):
            if isinstance(spec, PagedSpec):
                for known, sites in out:
                    if known == spec:
                        sites.append(site)
                        break
                else:
                    out.append((spec, [site]))
        return out

    def __init__(self, site_specs: Sequence[StateSpec], page_size: int, n_pages: Union[int, Sequence[int]],
                 n_slots: int):
        """`n_pages`: the pool size of every group, or one size per group (in the order of `groups_of`)."""
        if page_size <= 0 or page_size & (page_size - 1):
            raise ValueError(f"page size must be a power of two, got {page_size}")
        self._lib = N.host_library()
        self.page_size = page_size
        self.site_specs = list(site_specs)
        grouped = self.groups_of(self.site_specs)
        specs = [spec for spec, _ in grouped]
        sites_of = [sites for _, sites in grouped]
        self.group_of_site: Dict[int, int] = {site: g for g, sites in enumerate(sites_of) for site in sites}
        sizes = [int(n_pages)] * len(specs) if isinstance(n_pages, int) else [int(n) for n in n_pages]
        if len(sizes) != len(specs):
            raise ValueError(f"{len(sizes)} pool sizes were given for {len(specs)} groups")
        windows = (ctypes.c_int32 * max(1, len(specs)))(*[s.window or 0 for s in specs])
        pool_sizes = (ctypes.c_int32 * max(1, len(specs)))(*sizes)
        self._c = self._lib.imparo_cache_new(len(specs), windows, page_size, pool_sizes, n_slots)
        if not self._c:
            raise ValueError("the cache manager refused its sizes")
        self.groups: List[CacheGroup] = []
        for g, spec in enumerate(specs):
            pool = PagePool(0, _borrowed=self._lib.imparo_cache_group_pool(self._c, g))
            grp = CacheGroup(self, g, spec, pool, page_size)
            grp.sites = sites_of[g]
            self.groups.append(grp)
        self.fixed_sites = [s for s, spec in enumerate(self.site_specs) if isinstance(spec, FixedSpec)]
        self.n_slots = n_slots
        self.slots = PagePool(0, _borrowed=self._lib.imparo_cache_slot_pool(self._c))
        self._handles: Dict[Hashable, int] = {}
        self._names: Dict[int, Hashable] = {}
        self._next_handle = 1
        self.length = _PerRequest(self, self._lib.imparo_cache_length)
        self.slot_of = _PerRequest(self, self._lib.imparo_cache_slot)
        self._scratch = np.empty(1024, dtype=np.int32)

    def __del__(self):
        if getattr(self, "_c", None):
            self._lib.imparo_cache_delete(self._c)
            self._c = None

    def _h(self, req: Hashable) -> int:
        h = self._handles.get(req)
        if h is None or not self._lib.imparo_cache_is_live(self._c, h):
            raise CacheError(f"request {req!r} is not live")
        return h

    def handle(self, req: Hashable) -> int:
        """The 64-bit name the native side knows `req` by (given out on first
        asking, before the request is live, so that a scheduler can use it)."""
        h = self._handles.get(req)
        if h is None:
            h = self._handles[req] = self._next_handle
            self._next_handle += 1
            self._names[h] = req
        return h

    def name_of(self, handle: int) -> Hashable:
        return self._names[handle]

    def _live_names(self) -> List[Hashable]:
        return [r for r, h in self._handles.items() if self._lib.imparo_cache_is_live(self._c, h)]

    # ------------------------------------------------------------ requests
    def is_live(self, req: Hashable) -> bool:
        h = self._handles.get(req)
        return h is not None and bool(self._lib.imparo_cache_is_live(self._c, h))

    def admit(self, req: Hashable) -> int:
        """Takes a state slot for a new request; its tables start empty. The
        caller zeroes the slot's device state."""
        if self.is_live(req):
            raise CacheError(f"request {req!r} is already live")
        slot = self._lib.imparo_cache_admit(self._c, self.handle(req))
        if slot == N.E_OUT_OF_PAGES:
            raise OutOfPages(f"all {self.n_slots} request slots are in use")
        return slot

    def release(self, req: Hashable) -> None:
        self._lib.imparo_cache_release(self._c, self._h(req))
        self.forget(req)

    def forget(self, req: Hashable) -> None:
        """Drops the name of a request that is not live (any more)."""
        h = self._handles.get(req)
        if h is not None and not self._lib.imparo_cache_is_live(self._c, h):
            del self._handles[req]
            del self._names[h]

    # ------------------------------------------------------------ growth
    def pages_needed(self, req: Hashable, new_length: int) -> List[int]:
        """How many pages each group must add for the request to hold
        positions below `new_length`."""
        out = (ctypes.c_int32 * max(1, len(self.groups)))()
        self._lib.imparo_cache_pages_needed(self._c, self._h(req), new_length, out)
        return list(out[:len(self.groups)])

    def reserve(self, req: Hashable, new_length: int):
        """Allocates the pages for positions [length, new_length) in every
        group, all or nothing. What it took can be given back with `rollback`
        until the request's next `commit`."""
        rc = self._lib.imparo_cache_reserve(self._c, self._h(req), new_length)
        if rc == N.E_OUT_OF_PAGES:
            raise OutOfPages(f"request {req!r} needs pages for {new_length} positions and the pool "
                             f"has none left")
        if rc == N.E_SHRINK:
            raise CacheError(f"request {req!r} cannot shrink from {self.length[req]} to {new_length}")
        return req

    def rollback(self, req: Hashable, taken=None) -> None:
        self._lib.imparo_cache_rollback(self._c, self._h(req))

    def commit(self, req: Hashable, new_length: int) -> None:
        """The step ran: the request now holds `new_length` positions. Pages a
        window has passed are given back."""
        self._lib.imparo_cache_commit(self._c, self._h(req), new_length)

    def scramble(self, seed: int) -> None:
        for i, g in enumerate(self.groups):
            g.pool.scramble(seed + i)

    # ------------------------------------------------------------ views
    def table(self, group: int, req: Hashable) -> List[int]:
        h = self._h(req)
        n = self._lib.imparo_cache_table_len(self._c, group, h)
        if n > self._scratch.shape[0]:
            self._scratch = np.empty(2 * n, dtype=np.int32)
        self._lib.imparo_cache_table_copy(self._c, group, h, self._scratch.ctypes.data, self._scratch.shape[0])
        return self._scratch[:n].tolist()

    def table_len(self, group: int, req: Hashable) -> int:
        return self._lib.imparo_cache_table_len(self._c, group, self._h(req))

    def free_pages(self) -> List[int]:
        return [g.pool.n_free for g in self.groups]

    def held_pages(self, req: Hashable) -> List[int]:
        return [sum(1 for p in self.table(g, req) if p >= 0) for g in range(len(self.groups))]

    def check(self) -> None:
        """Every page is free or held by exactly one request; raises otherwise."""
        rc = self._lib.imparo_cache_check(self._c)
        if rc == N.E_SHARED_PAGE:
            raise CacheError("a page is held by two requests, or held and free")
        if rc == N.E_LOST_PAGE:
            raise CacheError("pages are lost: neither free nor held")
        if rc == N.E_SLOTS:
            raise CacheError("state slots are lost or held twice")

    # ------------------------------------------------------------ a step, as flat arrays
    def batch(self, requests: Sequence[Hashable], token_lists: Sequence[Sequence[int]],
              want_lists: Sequence[Sequence[int]]) -> "StepBatch":
        """The rows of a step as the native side takes them: handles, counts,
        and all token ids and wanted places end to end."""
        R = len(requests)
        b = StepBatch()
        b.requests = list(requests)
        b.reqs = np.fromiter(map(self.handle, requests), dtype=np.int64, count=R)
        b.n_tok = np.fromiter(map(len, token_lists), dtype=np.int32, count=R)
        b.n_want = np.fromiter(map(len, want_lists), dtype=np.int32, count=R)
        b.T, b.W = int(b.n_tok.sum()), int(b.n_want.sum())
        try:
            b.tokens = np.fromiter(chain.from_iterable(token_lists), dtype=np.int32, count=b.T)
            b.want = np.fromiter(chain.from_iterable(want_lists), dtype=np.int32, count=b.W)
        except (OverflowError, TypeError, ValueError) as e:
            raise CacheError(f"token ids and wanted places must be integers that fit 32 bits: {e}") from None
        b.new_slots = np.full(R, -1, dtype=np.int32)
        b.widest = 1
        b.device_tokens = None
        return b

    def begin_step(self, b: "StepBatch", vocab: int, max_position: int) -> Tuple[int, int]:
        """Checks the batch, admits its new requests and reserves every row's
        pages, all or nothing. Returns (0, -1) or (the native code of what is
        wrong, the row); raises OutOfPages. b.new_slots then names the slots
        whose device state the caller has to clear, b.widest the widest block
        table in pages."""
        info = np.zeros(3, dtype=np.int32)
        rc = self._lib.imparo_cache_begin_step(self._c, len(b.requests), b.reqs.ctypes.data, b.n_tok.ctypes.data,
                                               b.tokens.ctypes.data, b.n_want.ctypes.data, b.want.ctypes.data,
                                               vocab, max_position, b.new_slots.ctypes.data, info.ctypes.data)
        row = int(info[0])
        if rc == N.E_OUT_OF_PAGES:
            req = b.requests[row]
            if info[2]:
                raise OutOfPages(f"all {self.n_slots} request slots are in use")
            raise OutOfPages(f"request {req!r} needs pages for {int(b.n_tok[row])} more positions and the pool "
                             f"has none left")
        b.widest = int(info[1])
        return rc, row

    def abort_step(self, b: "StepBatch") -> None:
        self._lib.imparo_cache_abort_step(self._c, len(b.requests), b.reqs.ctypes.data, b.new_slots.ctypes.data)

    def end_step(self, b: "StepBatch") -> None:
        """The step ran: every row's request now holds its tokens; pages a window has passed are given back."""
        self._lib.imparo_cache_end_step(self._c, len(b.requests), b.reqs.ctypes.data, b.n_tok.ctypes.data)

    # ------------------------------------------------------------ a step's index arrays
    LAYOUT = ("T", "R", "W", "G", "P", "n_single", "n_multi", "max_seg_len", "max_context", "total")

    def pack(self, requests: Sequence[Hashable], token_lists: Sequence[Sequence[int]],
             want_lists: Sequence[Sequence[int]], table_width: int = 0) -> Tuple[np.ndarray, Dict[str, int]]:
        """One int32 array holding everything the kernels index by, laid out
        tokens | positions | row_of_token | seg_start | seg_len | slot | row
        lists | want | tables[group][row][page], and the sizes of its parts.
        Lengths are those before the step."""
        b = self.batch(requests, token_lists, want_lists)
        if table_width <= 0:
            b.widest = max([1] + [self._lib.imparo_cache_table_len(self._c, g, int(h))
                                  for h in b.reqs for g in range(len(self.groups))])
        return self.pack_batch(b, table_width)

    def pack_batch(self, b: "StepBatch", table_width: int = 0) -> Tuple[np.ndarray, Dict[str, int]]:
        R = len(b.requests)
        layout = np.zeros(len(self.LAYOUT), dtype=np.int32)
        P = table_width if table_width > 0 else b.widest
        capacity = 3 * b.T + 4 * R + b.W + len(self.groups) * R * P
        out = np.empty(capacity, dtype=np.int32)
        n = self._lib.imparo_cache_pack(self._c, R, b.reqs.ctypes.data, b.n_tok.ctypes.data, b.tokens.ctypes.data,
                                        b.n_want.ctypes.data, b.want.ctypes.data, table_width, out.ctypes.data,
                                        capacity, layout.ctypes.data)
        if n < 0:
            raise CacheError(f"packing the step failed with code {n}")
        return out[:n], dict(zip(self.LAYOUT, layout.tolist()))


class StepBatch:
    """The rows of one step as flat arrays (see CacheManager.batch)."""
    __slots__ = ("requests", "reqs", "n_tok", "n_want", "tokens", "want", "T", "W", "new_slots", "widest",
                 "device_tokens")     # device_tokens: (source vector, places in `tokens`, indices into the source) or None
