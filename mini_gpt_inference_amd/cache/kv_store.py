"""Device memory of the cache: page pools per cache group and per-request state pools."""

from __future__ import annotations

from typing import List, Sequence

import torch

from ..parts.model import CacheLayout
from .manager import GroupGeometry


class KVStore:
    """One tensor per group, [pools, 2 (keys, values; 1 in a joint group), pages, kv_heads, page_size, head_dim], in the
    compute dtype; one [max_requests, numel] float32 tensor per state binding.  With poison=True the
    pools start as NaN, so a kernel that reads a slot nobody wrote shows up in the logits."""

    def __init__(self, layout: CacheLayout, geometry: Sequence[GroupGeometry], max_requests: int,
                 dtype: torch.dtype, device: torch.device, poison: bool = False) -> None:
        assert len(geometry) == len(layout.groups)
        self.pools: List[torch.Tensor] = []
        fill = float("nan") if poison else 0.0
        for spec, geo in zip(layout.groups, geometry):
            # a joint group's pages hold one tensor that is both keys and values
            shape = (spec.n_pools, 1 if spec.joint else 2, geo.num_pages, spec.n_kv_head, geo.page_size, spec.head_dim)
            self.pools.append(torch.full(shape, fill, dtype=dtype, device=device))
        self.state_pools = [torch.full((max_requests, n), fill, dtype=torch.float32, device=device)
                            for n in layout.state_numels]

    def snapshot_states(self, slots: Sequence[int]) -> List[torch.Tensor]:
        """Copies of the given requests' rows of every state pool.  Pages take a step's keys and values
        a second time without harm; a state that the step has advanced must not be advanced again, so
        whoever runs a step's forward pass twice puts these back in between (restore_states)."""
        if not self.state_pools or not len(slots):
            return []
        index = torch.tensor(list(slots), dtype=torch.long, device=self.state_pools[0].device)
        return [index] + [pool.index_select(0, index) for pool in self.state_pools]

    def restore_states(self, saved: List[torch.Tensor]) -> None:
        if saved:
            for pool, rows in zip(self.state_pools, saved[1:]):
                pool.index_copy_(0, saved[0], rows)

    def k_pools(self, group: int) -> List[torch.Tensor]:
        p = self.pools[group]
        return [p[i, 0] for i in range(p.shape[0])]

    def v_pools(self, group: int) -> List[torch.Tensor]:
        p = self.pools[group]
        return [p[i, p.shape[1] - 1] for i in range(p.shape[0])]

    def bytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.pools + self.state_pools)
