"""What a mixer keeps for a request, and the memory for it.

A *need* is what ``Mixer.cache_need()`` returns.  It says how the cache manager accounts for it
and it owns its device memory: it allocates it, hands a mixer its view of it in a step, and
resets it when a request starts.  The engine never looks inside: a mixer with another kind of
cache (one latent vector per token, keys without values, a state of several tensors) brings a
need of its own, and no engine file changes.

Two ways of keeping:

  per token (``per_token = True``)   one entry for every position, kept in pages.  Needs that
      compare equal form a *group*: one pool of pages, one block table per request; every cache
      of the group is a *plane* of the same pages.  ``window`` = how many of the latest positions
      a query still reads (``None``: all); the manager hands back the pages a window has passed.
  per request (``per_token = False``)  memory of fixed size in the request's *slot*, zero when the
      request starts.

Interface (``units``: for a per-token need the pages of the pool + 2: unit 0 is the *null page*,
which nothing ever writes and which a table entry of -1 stands for (a kernel that reads a key
without a page reads zeros there), units 1.. are the allocator's pages, the last one is the spare
page where the rows that pad a batch read and write; the step's tables name units.  For a
per-request need: the slots + 1, the last one the spare slot):

  allocate(n_caches, units, page_size, device, dtype) -> store    anything the need likes
      (``page_size``: the entries of a page of this need's group)
  view(store, plane, ctx, group, writes) -> what the mixer's ``forward`` gets as ``cache``;
      ``ctx.block_tables[group]`` [requests, pages] and ``ctx.slots[group]`` [tokens] (the slot of
      the entry that holds each token's position: unit * entries per page + entry in the page) are
      the step's tables of a per-token group, ``ctx.seq_slots`` [requests] the slots
  bytes_per_token(dtype) -> int       per-token needs: for the measurement of cache traffic
  store_bytes(store) -> int
  reset(store, ctx)                   per-request needs: zero the slots ``ctx.reset_slots`` names
      (int32 [requests], -1 = leave alone) with work queued on the current stream
  clear_fresh(store, pages)           per-token needs: zero the units ``pages`` (int32 on the device,
      -1 = none) that the step has just taken from the pool, in every plane, before anything is
      written: what an earlier request left in a page (a NaN, an overflow) must not reach the
      request that gets the page next through a probability of zero times a stale value
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


class CacheNeed:
    per_token: bool = True
    window: Optional[int] = None
    # Per-token needs: how the positions of a request map to the entries of its pages.  One entry
    # holds ``tokens_per_entry`` consecutive positions (1: an entry a token; k: a mixer that keeps
    # one record per block of k tokens), and a page of this need's group has ``page_entries``
    # entries (None: the page size the cache was made with).  The manager counts pages, and the
    # step's tables name slots, by these numbers; groups with other numbers have pools of their own.
    tokens_per_entry: int = 1
    page_entries: Optional[int] = None

    def allocate(self, n_caches: int, units: int, page_size: int, device, dtype):
        raise NotImplementedError

    def view(self, store, plane: int, ctx, group: Optional[int], writes: bool):
        raise NotImplementedError

    def bytes_per_token(self, dtype) -> int:
        return 0

    def store_bytes(self, store) -> int:
        return 0

    def reset(self, store, ctx) -> None:
        """Per-request needs only."""

    def clear_fresh(self, store, pages) -> None:
        """Per-token needs only."""


class LayerCache:
    """What the engine's own needs hand a mixer in one step.

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


@dataclass(frozen=True)
class PagedNeed(CacheNeed):
    """One entry per token and layer: ``n_kv_heads * head_dim`` keys and as many values, in the
    compute dtype.  Keys lie row-major in a page, values transposed (a page of values is
    [head_dim, page_size]), which is how the attention kernels read them."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    per_token = True

    def __post_init__(self):
        if self.n_kv_heads < 1 or self.head_dim < 1:
            raise ValueError("PagedNeed: sizes must be positive")
        if self.window is not None and self.window < 1:
            raise ValueError("PagedNeed: window must be >= 1")

    def allocate(self, n_caches, units, page_size, device, dtype):
        import torch

        # The pools start as zeros, a page is zeroed again when a request takes it, and the null
        # page is never written: a probability of zero times a slot that no token of this request
        # has filled is zero, whatever an earlier request computed.
        k = torch.zeros((n_caches, units, self.n_kv_heads, page_size, self.head_dim), dtype=dtype, device=device)
        v = torch.zeros((n_caches, units, self.n_kv_heads, self.head_dim, page_size), dtype=dtype, device=device)
        return k, v, page_size

    def view(self, store, plane, ctx, group, writes):
        lc = LayerCache()
        lc.writes = writes
        lc.k_pool, lc.v_pool, lc.page_size = store[0][plane], store[1][plane], store[2]
        lc.block_tables, lc.slots, lc.group = ctx.block_tables[group], ctx.slots[group], group
        return lc

    def clear_fresh(self, store, pages) -> None:
        from .. import ops

        ops.zero_pages(store[0], store[1], pages)

    def bytes_per_token(self, dtype) -> int:
        import torch

        return 2 * self.n_kv_heads * self.head_dim * torch.empty((), dtype=dtype).element_size()

    def store_bytes(self, store) -> int:
        return sum(t.numel() * t.element_size() for t in store[:2])


@dataclass(frozen=True)
class StateNeed(CacheNeed):
    """A tensor of fixed ``shape`` per request and layer (torch dtype name, e.g. 'float32')."""

    shape: Tuple[int, ...]
    dtype: str = "float32"
    per_token = False

    def allocate(self, n_caches, units, page_size, device, dtype):
        import torch

        return torch.zeros((units, *self.shape), dtype=getattr(torch, self.dtype), device=device)

    def view(self, store, plane, ctx, group, writes):
        lc = LayerCache()
        lc.writes = writes
        lc.state = store
        return lc

    def store_bytes(self, store) -> int:
        return store.numel() * store.element_size()

    def reset(self, store, ctx) -> None:
        from .. import ops

        ops.zero_rows(store, ctx.reset_slots)
