"""The device memory behind the cache manager's pages and slots.

Per cache site with a paged spec: a K pool [n_pages, kv_heads, page_size,
head_dim], so one kv head's rows of a page are contiguous, and a V pool of the
same layout or, where the matrix-core attention kernels apply (bfloat16, pages
of at least 16), transposed inside the page: [n_pages, kv_heads, head_dim,
page_size]. Per site with a fixed spec: [n_slots, *shape] float32.
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
        self.kv: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self.v_transposed: Dict[int, bool] = {}
        self.fixed: Dict[int, torch.Tensor] = {}
        for site, spec in enumerate(manager.site_specs):
            if isinstance(spec, PagedSpec):
                g = manager.groups[manager.group_of_site[site]]
                shape = (g.pool.n_pages, spec.kv_heads, manager.page_size, spec.head_dim)
                vt = ops.mfma_attention_supported(dtype, manager.page_size, spec.head_dim)
                v_shape = (shape[0], shape[1], shape[3], shape[2]) if vt else shape
                self.v_transposed[site] = vt
                self.kv[site] = (torch.zeros(shape, dtype=dtype, device=device),
                                 torch.zeros(v_shape, dtype=dtype, device=device))
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
