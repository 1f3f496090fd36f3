"""Device memory behind the cache manager's bookkeeping."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .manager import CacheManager


@dataclass
class PagedLayerView:
    """What a mixer sees of one paged cache layer: the layer's pool of every tensor its
    cache spec names, [num_pages, *page shape] each, also as attributes (``.k``, ``.v`` for
    keys and values in pages of [Hkv, page_size, D])."""
    tensors: Dict[str, torch.Tensor]
    group: int                 # index into StepContext.groups
    page_size: int
    writable: bool
    kind: str = "paged"

    def __getattr__(self, name):               # (reached only for names that are no field)
        try:
            return self.__dict__["tensors"][name]
        except KeyError:
            raise AttributeError(f"this cache layer keeps no tensor {name!r}") from None


@dataclass
class StateLayerView:
    """What a mixer sees of one fixed-size-state cache layer."""
    state: torch.Tensor        # [max_num_seqs + 1, *shape], row = the request's state slot; the
                               # last row is the padding slot (rows that pad a replayed step)
    group: int
    writable: bool
    kind: str = "state"


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class CacheStorage:
    """Per paged group and per tensor of its spec a pool [layers, num_pages, *page shape]
    (for keys and values [layers, num_pages, Hkv, page_size, D]; the reference keeps one
    [max_tokens, 2*Hkv, D] tensor per layer, lite_llama/executor/mem_manager.py:166-168), and
    one [layers, max_num_seqs + 1, *shape] tensor per state group (the last row is the
    padding slot of the manager)."""

    def __init__(self, manager: CacheManager, dtype: torch.dtype, device):
        self.manager = manager
        self.paged_pools: List[Dict[str, torch.Tensor]] = []
        self.state_pools: List[torch.Tensor] = []
        for g in manager.paged:
            self.paged_pools.append({
                t.name: torch.zeros((len(g.layers), g.pool.num_pages) + t.page_shape(g.page_size),
                                    dtype=t.dtype or dtype, device=device)
                for t in g.spec.tensors})
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
            return PagedLayerView({name: pool[i] for name, pool in self.paged_pools[g].items()}, g,
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
            size = _element_size(g.spec.dtype or dtype)
            n = 1
            for d in g.spec.shape:
                n *= int(d)
            total += len(g.layers) * (manager.max_num_seqs + 1) * n * size
        return total

    @staticmethod
    def bytes_per_page(manager: CacheManager, dtype: torch.dtype) -> int:
        """Bytes that one more page of every paged group takes (all layers, all tensors)."""
        total = 0
        for g in manager.paged:
            for t in g.spec.tensors:
                n = g.page_size
                for d in t.shape:
                    n *= int(d)
                total += len(g.layers) * n * _element_size(t.dtype or dtype)
        return total
