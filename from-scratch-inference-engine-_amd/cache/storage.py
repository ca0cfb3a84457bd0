"""Device side of the cache: what every need allocated, and the views the mixers get."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Tuple

from .manager import CacheManager
from .needs import CacheNeed, LayerCache  # noqa: F401  (LayerCache is also named from here)


@dataclass
class CacheLayout:
    """Which cache (one per writing call of the model's schedule) lives where.

    ``paged_groups[g]`` is the per-token need shared by the caches ``group_caches[g]`` (their order
    is the order of planes in the group's pool); ``state_caches`` maps a cache id to its
    per-request need."""

    paged_groups: List[CacheNeed]
    group_caches: List[List[int]]
    state_caches: Dict[int, CacheNeed]

    def locate(self, cache_id: int) -> Tuple[int, int]:
        for g, ids in enumerate(self.group_caches):
            if cache_id in ids:
                return g, ids.index(cache_id)
        raise KeyError(f"cache {cache_id} is not paged")


class CacheStorage:
    """Asks every need for its memory and for the views; knows no layout itself.

    A pool has two pages more than its allocator: unit 0 is the null page (never written; what a
    table entry of -1 reads), the allocator's page p is unit p + 1, and the last unit is the spare
    page, which, like the last state slot, belongs to no request: the rows that pad a batch to a
    captured graph's size read and write there.  ``spare_pages`` names the spare page as the
    allocator would (its number of pages): the step's tables turn page ids into units."""

    def __init__(self, layout: CacheLayout, manager: CacheManager, device, dtype):
        self.layout = layout
        self.page_size = manager.page_size
        self.device = device
        self.dtype = dtype
        self.spare_pages: List[int] = [manager.allocators[g].num_pages for g in range(len(layout.paged_groups))]
        self.spare_slot = manager.max_requests
        # positions that a page of each group holds (the filler rows of a padded batch need as many
        # entries of the spare page in their tables as their tokens span)
        self.tokens_per_page: List[int] = [manager.tokens_per_page(g) for g in range(len(layout.paged_groups))]
        self.group_stores = [need.allocate(len(layout.group_caches[g]), self.spare_pages[g] + 2,
                                           manager.entries_per_page[g], device, dtype)
                             for g, need in enumerate(layout.paged_groups)]
        self.state_stores = {cid: need.allocate(1, manager.max_requests + 1, self.page_size, device, dtype)
                             for cid, need in layout.state_caches.items()}

    def bytes(self) -> int:
        return (sum(need.store_bytes(s) for need, s in zip(self.layout.paged_groups, self.group_stores))
                + sum(self.layout.state_caches[cid].store_bytes(s) for cid, s in self.state_stores.items()))

    def reset_states(self, ctx) -> None:
        """Zero the per-request memory of the requests that start in this step (queued on the
        stream like the rest of the step, from the step's own tables)."""
        for cid, store in self.state_stores.items():
            self.layout.state_caches[cid].reset(store, ctx)

    def clear_fresh(self, ctx) -> None:
        """Zero the pages that this step's requests have just taken from the pools."""
        for g, need in enumerate(self.layout.paged_groups):
            if ctx.fresh_pages[g] is not None:
                need.clear_fresh(self.group_stores[g], ctx.fresh_pages[g])

    def view(self, cache_id: int, ctx, writes: bool):
        if cache_id in self.state_stores:
            return self.layout.state_caches[cache_id].view(self.state_stores[cache_id], 0, ctx, None, writes)
        g, plane = self.layout.locate(cache_id)
        return self.layout.paged_groups[g].view(self.group_stores[g], plane, ctx, g, writes)
