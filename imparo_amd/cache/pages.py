"""Host-side bookkeeping of the cache: pages, block tables, state slots.

Nothing here touches the GPU; the tensors the pages index live in
`imparo_amd.cache.storage`.

Allocation always takes the lowest free page, so which pages a request gets
is a function of which pages are free and never of history; freeing a page
twice is an error. The reference's block allocator keeps the same two rules
(/root/reference/crates/imparo-kv/src/alloc.rs:1-11,51-75).
"""
from __future__ import annotations

import heapq
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple, Union


class OutOfPages(RuntimeError):
    """The pool cannot give the pages (or the slot) a step needs."""


class CacheError(RuntimeError):
    """Misuse of the cache manager: a page freed twice, an unknown request."""


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages < 0:
            raise ValueError("a pool cannot have a negative number of pages")
        self.n_pages = n_pages
        self._place: Optional[List[int]] = None   # rank -> page, when placement is scrambled
        self._rank: Optional[List[int]] = None
        self._heap = list(range(n_pages))
        self._free = [True] * n_pages
        self.n_free = n_pages
        self.high_water = 0      # one past the highest page ever handed out

    def alloc(self) -> int:
        if self.n_free == 0:
            raise OutOfPages("no free page")
        page = heapq.heappop(self._heap)
        if self._place is not None:
            page = self._place[page]
        self._free[page] = False
        self.n_free -= 1
        self.high_water = max(self.high_water, page + 1)
        return page

    def free(self, page: int) -> None:
        if not 0 <= page < self.n_pages:
            raise CacheError(f"page {page} is outside the pool of {self.n_pages}")
        if self._free[page]:
            raise CacheError(f"page {page} freed twice")
        self._free[page] = True
        self.n_free += 1
        heapq.heappush(self._heap, page if self._rank is None else self._rank[page])

    def scramble(self, seed: int) -> None:
        """Permutes which physical page each allocation rank maps to, so that
        block tables are not the identity. Only on an untouched pool. Output
        must not depend on it: placement is invisible
        (/root/reference/crates/imparo-kv/src/resident.rs:56-99)."""
        if self.n_free != self.n_pages:
            raise CacheError("placement can only be scrambled while every page is free")
        import random
        place = list(range(self.n_pages))
        random.Random(seed).shuffle(place)
        self._place = place
        self._rank = [0] * self.n_pages
        for rank, page in enumerate(place):
            self._rank[page] = rank

    def is_free(self, page: int) -> bool:
        return self._free[page]


@dataclass(frozen=True)
class PagedSpec:
    """State that grows with the context: keys and values per position.
    `window` None keeps every position; a number keeps only that many."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedSpec:
    """State of a fixed size per request (a conv history, a recurrent matrix)."""
    shape: Tuple[int, ...]


StateSpec = Union[PagedSpec, FixedSpec, None]


class CacheGroup:
    """The cache sites that share one paged spec: one pool of pages, one block
    table per request, the same page ids on every site of the group."""

    def __init__(self, spec: PagedSpec, sites: Sequence[int], n_pages: int, page_size: int):
        self.spec = spec
        self.sites = list(sites)
        self.page_size = page_size
        self.pool = PagePool(n_pages)
        self.tables: Dict[Hashable, List[int]] = {}

    def first_needed_page(self, next_position: int) -> int:
        """The lowest logical page a query at `next_position` or later reads."""
        if self.spec.window is None:
            return 0
        return max(0, next_position + 1 - self.spec.window) // self.page_size


class CacheManager:
    """Pages and slots of every live request.

    A request is admitted (gets a state slot, empty tables), grows by
    `reserve` (pages for the positions a step will write) followed by
    `commit` (the step ran) or `rollback` (it did not), and leaves by
    `release`, which gives back everything it holds.
    """

    def __init__(self, site_specs: Sequence[StateSpec], page_size: int, n_pages: int, n_slots: int):
        if page_size <= 0 or page_size & (page_size - 1):
            raise ValueError(f"page size must be a power of two, got {page_size}")
        self.page_size = page_size
        self.site_specs = list(site_specs)
        self.groups: List[CacheGroup] = []
        self.group_of_site: Dict[int, int] = {}
        by_spec: Dict[PagedSpec, int] = {}
        for site, spec in enumerate(self.site_specs):
            if isinstance(spec, PagedSpec):
                if spec not in by_spec:
                    by_spec[spec] = len(self.groups)
                    self.groups.append(CacheGroup(spec, [], n_pages, page_size))
                g = by_spec[spec]
                self.groups[g].sites.append(site)
                self.group_of_site[site] = g
        self.fixed_sites = [s for s, spec in enumerate(self.site_specs) if isinstance(spec, FixedSpec)]
        self.n_slots = n_slots
        self.slots = PagePool(n_slots)
        self.slot_of: Dict[Hashable, int] = {}
        self.length: Dict[Hashable, int] = {}

    # ------------------------------------------------------------ requests
    def is_live(self, req: Hashable) -> bool:
        return req in self.slot_of

    def admit(self, req: Hashable) -> int:
        """Takes a state slot for a new request; its tables start empty. The
        caller zeroes the slot's device state."""
        if req in self.slot_of:
            raise CacheError(f"request {req!r} is already live")
        try:
            slot = self.slots.alloc()
        except OutOfPages:
            raise OutOfPages(f"all {self.n_slots} request slots are in use") from None
        self.slot_of[req] = slot
        self.length[req] = 0
        for g in self.groups:
            g.tables[req] = []
        return slot

    def release(self, req: Hashable) -> None:
        if req not in self.slot_of:
            raise CacheError(f"request {req!r} is not live")
        for g in self.groups:
            for page in g.tables.pop(req):
                if page >= 0:
                    g.pool.free(page)
        self.slots.free(self.slot_of.pop(req))
        del self.length[req]

    # ------------------------------------------------------------ growth
    def pages_needed(self, req: Hashable, new_length: int) -> List[int]:
        """How many pages each group must add for the request to hold
        positions below `new_length`."""
        out = []
        for g in self.groups:
            table = g.tables[req]
            total = (new_length + self.page_size - 1) // self.page_size
            out.append(max(0, total - len(table)))
        return out

    def reserve(self, req: Hashable, new_length: int) -> List[Tuple[int, int]]:
        """Allocates the pages for positions [length, new_length) in every
        group, all or nothing. Returns what it took, for `rollback`."""
        if req not in self.slot_of:
            raise CacheError(f"request {req!r} is not live")
        if new_length < self.length[req]:
            raise CacheError(f"request {req!r} cannot shrink from {self.length[req]} to {new_length}")
        taken: List[Tuple[int, int]] = []
        try:
            for gi, g in enumerate(self.groups):
                table = g.tables[req]
                total = (new_length + self.page_size - 1) // self.page_size
                first = g.first_needed_page(self.length[req])
                while len(table) < total:
                    if len(table) < first:
                        table.append(-1)          # wholly behind the window: never needed
                        taken.append((gi, -1))
                        continue
                    page = g.pool.alloc()
                    table.append(page)
                    taken.append((gi, page))
        except OutOfPages:
            self._undo(req, taken)
            raise OutOfPages(f"request {req!r} needs pages for {new_length} positions and the pool "
                             f"has none left") from None
        return taken

    def _undo(self, req: Hashable, taken: List[Tuple[int, int]]) -> None:
        for gi, page in reversed(taken):
            table = self.groups[gi].tables[req]
            got = table.pop()
            assert got == page
            if page >= 0:
                self.groups[gi].pool.free(page)

    def rollback(self, req: Hashable, taken: List[Tuple[int, int]]) -> None:
        self._undo(req, taken)

    def commit(self, req: Hashable, new_length: int) -> None:
        """The step ran: the request now holds `new_length` positions. Pages a
        window has passed are given back."""
        self.length[req] = new_length
        for g in self.groups:
            if g.spec.window is None:
                continue
            table = g.tables[req]
            for idx in range(min(g.first_needed_page(new_length), len(table))):
                if table[idx] >= 0:
                    g.pool.free(table[idx])
                    table[idx] = -1

    def scramble(self, seed: int) -> None:
        for i, g in enumerate(self.groups):
            g.pool.scramble(seed + i)

    # ------------------------------------------------------------ views
    def table(self, group: int, req: Hashable) -> List[int]:
        return self.groups[group].tables[req]

    def free_pages(self) -> List[int]:
        return [g.pool.n_free for g in self.groups]

    def held_pages(self, req: Hashable) -> List[int]:
        return [sum(1 for p in g.tables[req] if p >= 0) for g in self.groups]

    def check(self) -> None:
        """Every page is free or held by exactly one request; raises otherwise."""
        for gi, g in enumerate(self.groups):
            seen: Dict[int, Hashable] = {}
            for req, table in g.tables.items():
                for page in table:
                    if page < 0:
                        continue
                    if page in seen:
                        raise CacheError(f"group {gi}: page {page} is held by {seen[page]!r} and {req!r}")
                    if g.pool.is_free(page):
                        raise CacheError(f"group {gi}: page {page} is held by {req!r} and free")
                    seen[page] = req
            if len(seen) + g.pool.n_free != g.pool.n_pages:
                raise CacheError(f"group {gi}: {g.pool.n_pages - len(seen) - g.pool.n_free} pages are lost")
        slots = list(self.slot_of.values())
        if len(set(slots)) != len(slots) or len(slots) + self.slots.n_free != self.n_slots:
            raise CacheError("state slots are lost or held twice")
