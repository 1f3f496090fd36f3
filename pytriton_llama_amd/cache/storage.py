"""Device memory behind the cache manager's bookkeeping."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch

from .manager import CacheManager


@dataclass
class PagedLayerView:
    """What a mixer sees of one paged cache layer."""
    k: torch.Tensor            # [num_pages, Hkv, page_size, D]
    v: torch.Tensor
    group: int                 # index into StepContext.groups
    page_size: int
    writable: bool
    kind: str = "paged"


@dataclass
class StateLayerView:
    """What a mixer sees of one fixed-size-state cache layer."""
    state: torch.Tensor        # [max_num_seqs + 1, *shape], row = the request's state slot; the
                               # last row is the padding slot (rows that pad a replayed step)
    group: int
    writable: bool
    kind: str = "state"


class CacheStorage:
    """Page pools [layers, num_pages, Hkv, page_size, D] for keys and for values
    per paged group (the reference keeps one [max_tokens, 2*Hkv, D] tensor per
    layer, lite_llama/executor/mem_manager.py:166-168), and one
    [layers, max_num_seqs + 1, *shape] tensor per state group (the last row is the padding
    slot of the manager)."""

    def __init__(self, manager: CacheManager, dtype: torch.dtype, device):
        self.manager = manager
        self.k_pools: List[torch.Tensor] = []
        self.v_pools: List[torch.Tensor] = []
        self.state_pools: List[torch.Tensor] = []
        for g in manager.paged:
            shape = (len(g.layers), g.pool.num_pages, g.spec.num_kv_heads, g.page_size,
                     g.spec.head_dim)
            self.k_pools.append(torch.zeros(shape, dtype=dtype, device=device))
            self.v_pools.append(torch.zeros(shape, dtype=dtype, device=device))
        for g in manager.states:
            shape = (len(g.layers), manager.max_num_seqs + 1) + tuple(g.spec.shape)
            self.state_pools.append(torch.zeros(shape, dtype=g.spec.dtype or dtype, device=device))

    def view(self, cache_layer: Optional[int], writable: bool = True):
        if cache_layer is None:
            return None
        home = self.manager.layer_home[cache_layer]
        if home is None:
            return None
        kind, g, i = home
        if kind == "paged":
            return PagedLayerView(self.k_pools[g][i], self.v_pools[g][i], g,
                                  self.manager.page_size, writable)
        return StateLayerView(self.state_pools[g][i], g, writable)

    def clear_slot(self, slot: int) -> None:
        """A new request starts from zero state."""
        for pool in self.state_pools:
            pool[:, slot].zero_()

    @staticmethod
    def state_bytes(manager: CacheManager, dtype: torch.dtype) -> int:
        """Bytes of the fixed-size state of all slots (what the state pools take whatever the
        number of pages)."""
        total = 0
        for g in manager.states:
            size = torch.empty((), dtype=g.spec.dtype or dtype).element_size()
            n = 1
            for d in g.spec.shape:
                n *= int(d)
            total += len(g.layers) * (manager.max_num_seqs + 1) * n * size
        return total

    @staticmethod
    def bytes_per_page(manager: CacheManager, dtype: torch.dtype) -> int:
        size = torch.empty((), dtype=dtype).element_size()
        return sum(2 * len(g.layers) * g.spec.num_kv_heads * g.page_size * g.spec.head_dim * size
                   for g in manager.paged)
