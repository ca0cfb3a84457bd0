"""Host side of the cache: who holds which page and which state slot.

The manager knows nothing of models.  It is built from *needs* (``cache.needs``): a per-token
need says that some layers keep one entry per token (all of them, or only a window of the
latest), a per-request need says that a layer keeps a fixed-size state per request.  Layers with
equal per-token needs form a *group*; a group has its own pool of pages, and each request has one
block table per group.  Of a need the manager reads the ``window`` only.
Device memory is not touched here (``cache.storage`` holds the tensors), so every decision
can be tested on the CPU.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, Iterable, List, Optional, Sequence, Tuple

from .allocator import OutOfPages, PageAllocator
from .needs import CacheNeed, PagedNeed, StateNeed  # noqa: F401  (PagedNeed and StateNeed are also named from here)


class NoFreeSlot(RuntimeError):
    """All per-request state slots are taken."""


@dataclass
class RequestCache:
    """What one live request holds: its state slot, its committed length, and per group a
    block table (page id for each page index; -1 where a window has passed and the page went
    back to the pool)."""

    request_id: Hashable
    slot: int
    length: int = 0
    tables: List[List[int]] = field(default_factory=list)
    closed: bool = False

    def pages_held(self, group: int) -> int:
        return sum(1 for p in self.tables[group] if p >= 0)


class CacheManager:
    def __init__(self, paged_groups: Sequence[CacheNeed], page_size: int,
                 num_pages, max_requests: int):
        """``num_pages``: one number for every group or one per group."""
        if page_size < 1:
            raise ValueError("CacheManager: page_size must be positive")
        if max_requests < 1:
            raise ValueError("CacheManager: max_requests must be positive")
        self.page_size = int(page_size)
        self.groups: List[CacheNeed] = list(paged_groups)
        # per group: entries in a page and positions in an entry (a need may state its own)
        self.entries_per_page = [int(getattr(n, "page_entries", None) or self.page_size) for n in self.groups]
        self.tokens_per_entry = [int(getattr(n, "tokens_per_entry", 1) or 1) for n in self.groups]
        if any(e < 1 for e in self.entries_per_page) or any(t < 1 for t in self.tokens_per_entry):
            raise ValueError("CacheManager: a group's page_entries and tokens_per_entry must be positive")
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.groups)
        if len(num_pages) != len(self.groups):
            raise ValueError("CacheManager: num_pages must match the number of groups")
        self.allocators = [PageAllocator(int(n)) for n in num_pages]
        self.max_requests = int(max_requests)
        self._free_slots = list(range(self.max_requests - 1, -1, -1))
        self._live: Dict[Hashable, RequestCache] = {}

    # ------------------------------------------------------------------ slots / requests
    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def live_requests(self) -> List[RequestCache]:
        return list(self._live.values())

    def open(self, request_id: Hashable) -> RequestCache:
        """Start a request: takes a state slot (its content is reset by the first step that
        runs the request at length 0), no pages yet."""
        if request_id in self._live:
            raise RuntimeError(f"CacheManager: request {request_id!r} is already open")
        if not self._free_slots:
            raise NoFreeSlot("CacheManager: no free state slot")
        rc = RequestCache(request_id=request_id, slot=self._free_slots.pop(),
                          tables=[[] for _ in self.groups])
        self._live[request_id] = rc
        return rc

    def get(self, request_id: Hashable) -> Optional[RequestCache]:
        return self._live.get(request_id)

    def close(self, rc: RequestCache) -> None:
        """Give back every page and the slot."""
        if rc.closed:
            raise RuntimeError(f"CacheManager: request {rc.request_id!r} closed twice")
        for g, table in enumerate(rc.tables):
            for page in table:
                if page >= 0:
                    self.allocators[g].free(page)
            table.clear()
        rc.length = 0
        rc.closed = True
        self._free_slots.append(rc.slot)
        del self._live[rc.request_id]

    # ------------------------------------------------------------------ pages
    def tokens_per_page(self, group: int = 0) -> int:
        """Positions that one page of ``group`` holds."""
        if not self.groups:
            return self.page_size
        return self.entries_per_page[group] * self.tokens_per_entry[group]

    @property
    def smallest_page_tokens(self) -> int:
        """The positions of the smallest page of any group: between two multiples of it no group
        needs a new page."""
        return min([self.tokens_per_page(g) for g in range(len(self.groups))] or [self.page_size])

    def pages_for(self, tokens: int, group: int = 0) -> int:
        return -(-tokens // self.tokens_per_page(group))

    def free_pages(self, group: int = 0) -> int:
        return self.allocators[group].num_free

    def first_needed_page(self, group: int, length: int) -> int:
        """Index of the first page that a query at position ``length`` (the next one) can still
        read in this group; earlier pages are dead."""
        window = self.groups[group].window
        if window is None:
            return 0
        return max(0, length - window + 1) // self.tokens_per_page(group)

    def new_pages_needed(self, rc: RequestCache, n_tokens: int) -> List[int]:
        """Pages each group must take from its pool to hold ``n_tokens`` more."""
        return [max(0, self.pages_for(rc.length + n_tokens, g) - len(t)) for g, t in enumerate(rc.tables)]

    def max_pages_held(self, total_tokens: int, portion: int) -> List[int]:
        """Upper bound of pages a request of ``total_tokens`` holds at once per group when it is
        fed in portions of at most ``portion`` tokens."""
        out = []
        for g, need in enumerate(self.groups):
            if need.window is None:
                out.append(self.pages_for(total_tokens, g))
            else:
                span = min(total_tokens, need.window + portion + self.tokens_per_page(g))
                out.append(min(self.pages_for(total_tokens, g), self.pages_for(span, g) + 1))
        return out

    def can_reserve(self, items: Iterable[Tuple[RequestCache, int]]) -> bool:
        """True if every item of one step can grow by its token count at the same time."""
        want = [0] * len(self.groups)
        for rc, n in items:
            for g, k in enumerate(self.new_pages_needed(rc, n)):
                want[g] += k
        return all(w <= a.num_free for w, a in zip(want, self.allocators))

    def reserve(self, rc: RequestCache, n_tokens: int) -> List[List[int]]:
        """Grow the block tables to hold ``length + n_tokens``.  Checks every group first, so a
        failure leaves the request as it was.  Returns, per group, the pages just taken."""
        if rc.closed:
            raise RuntimeError(f"CacheManager: request {rc.request_id!r} is closed")
        if n_tokens < 0:
            raise ValueError("CacheManager: negative token count")
        need = self.new_pages_needed(rc, n_tokens)
        for g, k in enumerate(need):
            if k > self.allocators[g].num_free:
                raise OutOfPages(
                    f"CacheManager: group {g} needs {k} pages for request {rc.request_id!r}, "
                    f"{self.allocators[g].num_free} free")
        fresh: List[List[int]] = [[] for _ in need]
        for g, k in enumerate(need):
            for _ in range(k):
                fresh[g].append(self.allocators[g].allocate())
            rc.tables[g].extend(fresh[g])
        return fresh

    def commit(self, rc: RequestCache, n_tokens: int) -> None:
        """The step wrote ``n_tokens`` entries: advance the length and give back the pages
        that no later query of a windowed group can read."""
        if rc.closed:
            raise RuntimeError(f"CacheManager: request {rc.request_id!r} is closed")
        if rc.tables and rc.length + n_tokens > min(len(t) * self.tokens_per_page(g) for g, t in enumerate(rc.tables)):
            raise RuntimeError("CacheManager: commit beyond the reserved pages")
        rc.length += n_tokens
        for g, table in enumerate(rc.tables):
            if self.groups[g].window is None:
                continue
            dead = min(self.first_needed_page(g, rc.length), len(table))
            for idx in range(dead):
                if table[idx] >= 0:
                    self.allocators[g].free(table[idx])
                    table[idx] = -1

    # ------------------------------------------------------------------ checks (tests, debug)
    def check_invariants(self) -> None:
        """No page lost, none held twice: per group, pages in tables + free pages = pool."""
        for g, alloc in enumerate(self.allocators):
            held: List[int] = []
            for rc in self._live.values():
                held.extend(p for p in rc.tables[g] if p >= 0)
            if len(held) != len(set(held)):
                raise AssertionError(f"group {g}: a page is held twice")
            if len(held) + alloc.num_free != alloc.num_pages:
                raise AssertionError(
                    f"group {g}: {len(held)} held + {alloc.num_free} free != {alloc.num_pages}")
            for p in held:
                if alloc.ref_count(p) != 1:
                    raise AssertionError(f"group {g}: held page {p} has ref count {alloc.ref_count(p)}")
        slots = [rc.slot for rc in self._live.values()]
        if len(slots) != len(set(slots)) or len(slots) + len(self._free_slots) != self.max_requests:
            raise AssertionError("state slots lost or held twice")


def pages_that_fit(free_bytes: int, bytes_per_token: int, page_size: int, fraction: float = 0.9,
                   reserve_bytes: int = 2 << 30) -> int:
    """Pages a pool can have when it may take ``fraction`` of ``free_bytes`` less ``reserve_bytes``
    (what a step's activations, the captured graphs and the library's workspaces need beside it);
    ``bytes_per_token`` is what one token holds in all groups and layers together.  At least one."""
    if bytes_per_token <= 0 or page_size <= 0:
        raise ValueError("pages_that_fit: bytes_per_token and page_size must be positive")
    room = int(free_bytes * fraction) - int(reserve_bytes)
    return max(1, room // (bytes_per_token * page_size))
