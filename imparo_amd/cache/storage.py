"""The device memory behind the cache manager's pages and slots.

Per cache site with a paged spec: one tensor per array the spec declares,
[n_pages of the site's group, *the array's page shape], in the engine's dtype
or in float32 as the array says. The layout inside a page is the mixer's
business: it declared it, and its kernels read it. Per site with a fixed spec:
[n_slots, *shape] float32, every slot at the spec's initial value.
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
        self.fixed: Dict[int, torch.Tensor] = {}
        for site, spec in enumerate(manager.site_specs):
            if isinstance(spec, PagedSpec):
                n_pages = manager.groups[manager.group_of_site[site]].pool.n_pages
                self.paged[site] = {
                    a.name: torch.zeros(a.shape(n_pages, manager.page_size),
                                        dtype=torch.float32 if a.float32 else dtype, device=device)
                    for a in spec.arrays}
            elif isinstance(spec, FixedSpec):
                self.fixed[site] = torch.full((manager.n_slots,) + tuple(spec.shape), float(spec.init),
                                              dtype=torch.float32, device=device)
        # what one launch needs to put a slot of every fixed site back to its initial value
        sites = sorted(self.fixed)
        self._reset_args = None
        if sites:
            self._reset_args = (
                torch.tensor([self.fixed[s].data_ptr() for s in sites], dtype=torch.int64, device=device),
                torch.tensor([self.fixed[s][0].numel() for s in sites], dtype=torch.int64, device=device),
                torch.tensor([float(manager.site_specs[s].init) for s in sites], dtype=torch.float32, device=device))

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
        for t in self.fixed.values():
            n += t.numel() * 4
        return n
