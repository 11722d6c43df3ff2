"""Device memory of the caches: page pools for paged groups, per-slot state tensors."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .manager import CacheManager


@dataclass
class CacheView:
    """What a mixer sees of one cache during a step."""
    cache_id: int
    group: int
    k: Optional[torch.Tensor] = None       # [num_pages, num_kv_heads, page_size, head_dim]
    v: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None   # [max_seqs, *state_shape]


class DeviceCache:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device, fill: float = 0.0):
        """``fill``: initial content of the pools (tests fill with NaN so that a read of a
        never-written place shows)."""
        self.manager = manager
        self.views: Dict[int, CacheView] = {}
        self.pools = {}
        for g in manager.groups:
            n = len(g.cache_ids)
            if g.paged:
                shape = (n, g.pool.num_pages, g.need.num_kv_heads, manager.page_size, g.need.head_dim)
                k = torch.full(shape, fill, dtype=dtype, device=device)
                v = torch.full(shape, fill, dtype=dtype, device=device)
                self.pools[g.index] = (k, v)
                for i, cid in enumerate(g.cache_ids):
                    self.views[cid] = CacheView(cid, g.index, k=k[i], v=v[i])
            else:
                sdt = g.need.state_dtype or torch.float32
                st = torch.zeros((n, manager.max_seqs) + tuple(g.need.state_shape), dtype=sdt, device=device)
                self.pools[g.index] = (st,)
                for i, cid in enumerate(g.cache_ids):
                    self.views[cid] = CacheView(cid, g.index, state=st[i])
        if any(not g.paged for g in manager.groups):
            # every admission, also a scheduler's or one after a pre-emption, starts from cleared state
            manager.on_admit.append(self.reset_slot)

    def reset_slot(self, slot: int) -> None:
        """Clear the fixed-size state of a slot that a new request takes over."""
        for g in self.manager.groups:
            if not g.paged:
                self.pools[g.index][0][:, slot].zero_()

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for ts in self.pools.values() for t in ts)
