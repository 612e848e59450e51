"""The device memory behind the cache manager's pages and slots.

Per cache site with a paged spec: a K and a V pool laid out
[n_pages, kv_heads, page_size, head_dim], so one kv head's rows of a page are
contiguous. Per site with a fixed spec: [n_slots, *shape] float32.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..kernels import ops
from .pages import CacheManager, FixedSpec, PagedSpec, StateSpec


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device: torch.device):
        self.manager = manager
        self.dtype = dtype
        self.device = device
        self.kv: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self.fixed: Dict[int, torch.Tensor] = {}
        for site, spec in enumerate(manager.site_specs):
            if isinstance(spec, PagedSpec):
                g = manager.groups[manager.group_of_site[site]]
                shape = (g.pool.n_pages, spec.kv_heads, manager.page_size, spec.head_dim)
                self.kv[site] = (torch.zeros(shape, dtype=dtype, device=device),
                                 torch.zeros(shape, dtype=dtype, device=device))
            elif isinstance(spec, FixedSpec):
                self.fixed[site] = torch.zeros((manager.n_slots,) + tuple(spec.shape),
                                               dtype=torch.float32, device=device)

    def zero_slot(self, slot: int) -> None:
        """A request that has seen nothing starts from zero state."""
        for t in self.fixed.values():
            ops.fill_f32(t[slot], 0.0)

    def bytes(self) -> int:
        n = 0
        for k, v in self.kv.values():
            n += k.numel() * k.element_size() * 2
        for t in self.fixed.values():
            n += t.numel() * 4
        return n
