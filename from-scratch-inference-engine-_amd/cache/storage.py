"""Device side of the cache: the pools of pages and the state slots."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .manager import CacheManager, PagedNeed, StateNeed


@dataclass
class CacheLayout:
    """Which cache (one per writing call of the model's schedule) lives where.

    ``paged_groups[g]`` is the need shared by the caches ``group_caches[g]`` (their order is the
    order of planes in the group's pool); ``state_caches`` maps a cache id to its state need."""

    paged_groups: List[PagedNeed]
    group_caches: List[List[int]]
    state_caches: Dict[int, StateNeed]

    def locate(self, cache_id: int) -> Tuple[int, int]:
        for g, ids in enumerate(self.group_caches):
            if cache_id in ids:
                return g, ids.index(cache_id)
        raise KeyError(f"cache {cache_id} is not paged")


class LayerCache:
    """What a mixer sees of the cache in one step.

    Paged: ``k_pool`` [pages + 1, kv_heads, page_size, head_dim] and ``v_pool`` [pages + 1, kv_heads,
    head_dim, page_size] of this layer (the last page is the spare one of padding rows),
    ``block_tables`` int32 [requests in the step, pages] (-1 = no page), ``slots`` int32 [tokens]
    (where each token's entry goes), ``page_size``, and ``writes`` (False when this call only
    reads a cache that another call fills).
    State: ``state`` [max_requests + 1, *shape]; the step's ``ctx.seq_slots`` index it."""

    __slots__ = ("k_pool", "v_pool", "block_tables", "slots", "page_size", "writes", "state", "group")

    def __init__(self):
        self.k_pool = self.v_pool = self.block_tables = self.slots = self.state = None
        self.page_size = 0
        self.writes = True
        self.group = -1


class CacheStorage:
    def __init__(self, layout: CacheLayout, manager: CacheManager, device, dtype: torch.dtype):
        self.layout = layout
        self.page_size = manager.page_size
        self.device = device
        self.dtype = dtype
        # per group: keys [caches, pages + 1, kv_heads, page_size, head_dim] and values, transposed
        # within a page, [caches, pages + 1, kv_heads, head_dim, page_size].  The last page of a
        # pool and the last state slot belong to no request (the allocators do not know them):
        # they are where the rows that pad a batch to a captured graph's size read and write.
        self.k_pools: List[torch.Tensor] = []
        self.v_pools: List[torch.Tensor] = []
        self.spare_pages: List[int] = []
        for g, need in enumerate(layout.paged_groups):
            n_pages = manager.allocators[g].num_pages
            n_caches = len(layout.group_caches[g])
            self.spare_pages.append(n_pages)
            self.k_pools.append(torch.zeros((n_caches, n_pages + 1, need.n_kv_heads, self.page_size, need.head_dim),
                                            dtype=dtype, device=device))
            self.v_pools.append(torch.zeros((n_caches, n_pages + 1, need.n_kv_heads, need.head_dim, self.page_size),
                                            dtype=dtype, device=device))
        self.spare_slot = manager.max_requests
        self.states: Dict[int, torch.Tensor] = {}
        for cid, need in layout.state_caches.items():
            self.states[cid] = torch.zeros((manager.max_requests + 1, *need.shape),
                                           dtype=getattr(torch, need.dtype), device=device)

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k_pools + self.v_pools + list(self.states.values()))

    def reset_states(self, slots: Sequence[int]) -> None:
        """Zero the state slots of requests that start in this step."""
        if not slots or not self.states:
            return
        idx = torch.tensor(list(slots), dtype=torch.int64, device=self.device)
        for t in self.states.values():
            t.index_fill_(0, idx, 0)

    def view(self, cache_id: int, ctx, writes: bool) -> LayerCache:
        lc = LayerCache()
        lc.writes = writes
        if cache_id in self.states:
            lc.state = self.states[cache_id]
            return lc
        g, plane = self.layout.locate(cache_id)
        lc.k_pool, lc.v_pool = self.k_pools[g][plane], self.v_pools[g][plane]
        lc.block_tables = ctx.block_tables[g]
        lc.slots = ctx.slots[g]
        lc.page_size = self.page_size
        lc.group = g
        return lc
