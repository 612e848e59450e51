"""The device memory behind the cache manager's pages and slots.

Per cache site with a paged spec: one tensor per array the spec declares,
[n_pages of the site's group, *the array's page shape], in the engine's dtype
or in float32 as the array says. The layout inside a page is the mixer's
business: it declared it, and its kernels read it. Per site with a fixed spec:
one tensor [n_slots, *shape] per array the spec declares, in the array's
dtype, every slot at the array's initial value.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from ..kernels import ops
from .pages import CacheManager, FixedSpec, PagedSpec


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device: torch.device):
        self.manager = manager
        self.dtype = dtype
        self.device = device
        self.paged: Dict[int, Dict[str, torch.Tensor]] = {}
        self.fixed: Dict[int, torch.Tensor] = {}                    # a site's one array, or its array named "state"
        self.fixed_arrays: Dict[int, Dict[str, torch.Tensor]] = {}   # every array of a site, by name
        for site, spec in enumerate(manager.site_specs):
            if isinstance(spec, PagedSpec):
                n_pages = manager.groups[manager.group_of_site[site]].pool.n_pages
                self.paged[site] = {
                    a.name: torch.zeros(a.shape(n_pages, manager.page_size),
                                        dtype=torch.float32 if a.float32 else dtype, device=device)
                    for a in spec.arrays}
            elif isinstance(spec, FixedSpec):
                kinds = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32, "engine": dtype}
                arrays = {a.name: torch.full((manager.n_slots,) + tuple(a.shape), a.init, dtype=kinds[a.dtype],
                                             device=device) for a in spec.all_arrays()}
                self.fixed_arrays[site] = arrays
                if len(arrays) == 1 or "state" in arrays:
                    self.fixed[site] = arrays.get("state", next(iter(arrays.values())))
        # What one launch needs to put a slot of every fixed array back to its initial value: the fill
        # writes 32-bit words, so an array of another width starts from zero (all bits clear in any
        # dtype) and takes a whole number of words per slot.
        resets = []
        for site in sorted(self.fixed_arrays):
            for a in manager.site_specs[site].all_arrays():
                t = self.fixed_arrays[site][a.name]
                per_slot = t[0].numel() * t.element_size()
                if per_slot % 4:
                    raise ValueError(f"site {site}, state array {a.name!r}: a slot of {per_slot} bytes is no whole "
                                     f"number of 32-bit words")
                resets.append((t.data_ptr(), per_slot // 4, float(a.init)))
        self._reset_args = None
        if resets:
            self._reset_args = (
                torch.tensor([r[0] for r in resets], dtype=torch.int64, device=device),
                torch.tensor([r[1] for r in resets], dtype=torch.int64, device=device),
                torch.tensor([r[2] for r in resets], dtype=torch.float32, device=device))

    @property
    def kv(self) -> Dict[int, Tuple[torch.Tensor, torch.Tensor]]:
        """The sites that keep arrays named k and v, as pairs."""
        return {site: (arrays["k"], arrays["v"]) for site, arrays in self.paged.items()
                if "k" in arrays and "v" in arrays}

    def reset_slot(self, slot: int) -> None:
        """A request that has seen nothing starts from every site's initial state: one launch."""
        if self._reset_args is not None:
            ops.fill_sites(*self._reset_args, slot)

    def bytes(self) -> int:
        n = 0
        for arrays in self.paged.values():
            n += sum(t.numel() * t.element_size() for t in arrays.values())
        for arrays in self.fixed_arrays.values():
            n += sum(t.numel() * t.element_size() for t in arrays.values())
        return n
