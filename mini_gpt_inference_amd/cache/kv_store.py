"""Device memory of the cache: page pools per cache group and per-request state pools."""

from __future__ import annotations

from typing import List, Sequence

import torch

from ..parts.model import CacheLayout
from .manager import GroupGeometry


class KVStore:
    """One tensor per group, [pools, 2 (keys, values), pages, kv_heads, page_size, head_dim], in the
    compute dtype; one [max_requests, numel] float32 tensor per state binding.  With poison=True the
    pools start as NaN, so a kernel that reads a slot nobody wrote shows up in the logits."""

    def __init__(self, layout: CacheLayout, geometry: Sequence[GroupGeometry], max_requests: int,
                 dtype: torch.dtype, device: torch.device, poison: bool = False) -> None:
        assert len(geometry) == len(layout.groups)
        self.pools: List[torch.Tensor] = []
        fill = float("nan") if poison else 0.0
        for spec, geo in zip(layout.groups, geometry):
            shape = (spec.n_pools, 2, geo.num_pages, spec.n_kv_head, geo.page_size, spec.head_dim)
            self.pools.append(torch.full(shape, fill, dtype=dtype, device=device))
        self.state_pools = [torch.zeros((max_requests, n), dtype=torch.float32, device=device)
                            for n in layout.state_numels]

    def k_pools(self, group: int) -> List[torch.Tensor]:
        p = self.pools[group]
        return [p[i, 0] for i in range(p.shape[0])]

    def v_pools(self, group: int) -> List[torch.Tensor]:
        p = self.pools[group]
        return [p[i, 1] for i in range(p.shape[0])]

    def bytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.pools + self.state_pools)
