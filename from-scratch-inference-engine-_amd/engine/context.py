"""What one step looks like to the parts: the tokens of the batch and their index tables.

The host collects every int32 table of the step (token ids, positions, block tables, cache slots,
attention work items, ...) into one pinned buffer and sends it with one copy; the parts see
device views of it."""

from __future__ import annotations

from dataclasses import dataclass, field
from types import SimpleNamespace
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places among them whose logits
    are wanted."""

    cache: RequestCache
    tokens: Sequence[int]
    want: Sequence[int] = ()
    # set by the step function: per group, the pages it has just reserved for these tokens
    fresh: Sequence[Sequence[int]] = ()


def filler_entry(storage, n_tokens: int):
    """Stands in a batch for a request that does not exist: ``n_tokens`` tokens of id 0 from
    position 0 that want no logits (or, with one token, its own), whose cache is the spare page
    of every pool, over and over, and the spare state slot.  Nothing a request reads is written."""
    spare = SimpleNamespace(length=0, slot=storage.spare_slot,
                            tables=[[p] * max(1, -(-n_tokens // per_page))
                                    for p, per_page in zip(storage.spare_pages, storage.tokens_per_page)],
                            request_id="(filler)")
    return SimpleNamespace(cache=spare, tokens=(0,) * n_tokens, want=())


def padded_tokens(n: int) -> int:
    """Rows of a step that is not a decode step, once filled up (done while the library's kernels
    are chosen by timing): up to 64 as they are, then 128, then the next multiple of 256 where that
    adds at most a fifth (or 64 rows).  Only these counts are timed (a count costs seconds the first
    time it comes), and a timed choice is up to a fifth faster than the library's own; without the
    timing the filled-up step is no faster than the step as it is."""
    if n <= 64:
        return n
    if n <= 128:
        return 128
    up = -(-n // 256) * 256
    return up if up - n <= max(64, n // 5) else n


class HostBatch:
    """Host view of the step, in the order of the entries."""

    def __init__(self, entries: Sequence[StepEntry], page_size: int = 0, compute_dtype=None):
        self.page_size = page_size
        self.compute_dtype = compute_dtype
        self.pad = None  # set for a step that replays a captured graph: tables padded to fixed sizes
        self.n_seqs = len(entries)
        self.q_lens = [len(e.tokens) for e in entries]
        self.past_lens = [e.cache.length for e in entries]
        self.q_starts = [0]
        for n in self.q_lens:
            self.q_starts.append(self.q_starts[-1] + n)
        self.n_tokens = self.q_starts[-1]
        self.seq_slots = [e.cache.slot for e in entries]
        # the slots of the requests that start in this step (their per-request memory is reset), -1 for the others
        self.reset_slots = [e.cache.slot if e.cache.length == 0 else -1 for e in entries]
        self.token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64).reshape(-1) for e in entries]
                                        ) if entries else np.zeros(0, np.int64)
        self.positions = np.concatenate(
            [np.arange(p, p + n, dtype=np.int32) for p, n in zip(self.past_lens, self.q_lens)]
        ) if entries else np.zeros(0, np.int32)
        self.want_rows = np.asarray([self.q_starts[i] + w for i, e in enumerate(entries) for w in e.want],
                                    dtype=np.int32)


class _Packer:
    """Collects int32 arrays; one pinned buffer, one copy."""

    ALIGN = 4  # ints: every table starts on 16 bytes

    def __init__(self):
        self._arrays: List[np.ndarray] = []
        self._offsets: List[int] = []
        self._total = 0

    def add(self, array: np.ndarray) -> int:
        array = np.ascontiguousarray(array, dtype=np.int32)
        self._arrays.append(array)
        self._offsets.append(self._total)
        self._total += -(-max(array.size, 1) // self.ALIGN) * self.ALIGN
        return len(self._arrays) - 1

    @property
    def total(self) -> int:
        return self._total

    def upload(self, staging: "PinnedStaging", device, into: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
        """Copy everything to the device in one go; ``into`` = an existing buffer of the same
        layout (a captured graph reads it), else a new one."""
        host = staging.acquire(self._total)
        flat = host.numpy()
        for a, off in zip(self._arrays, self._offsets):
            flat[off:off + a.size] = a.reshape(-1)
        if into is None:
            into = torch.empty((self._total,), dtype=torch.int32, device=device)
        elif into.numel() != self._total:
            raise RuntimeError("step tables do not have the layout of the captured graph")
        into.copy_(host[:self._total], non_blocking=True)
        staging.release()
        return [into[off:off + a.size].view(a.shape) for a, off in zip(self._arrays, self._offsets)]


class PinnedStaging:
    """A pinned host buffer reused from step to step; an event guards it until the copy that
    read it has run."""

    def __init__(self):
        self._buf: Optional[torch.Tensor] = None
        self._event: Optional[torch.cuda.Event] = None

    def acquire(self, n_ints: int) -> torch.Tensor:
        if self._event is not None:
            self._event.synchronize()
        if self._buf is None or self._buf.numel() < n_ints:
            self._buf = torch.empty((max(n_ints, 1 << 14),), dtype=torch.int32, pin_memory=True)
        return self._buf

    def release(self) -> None:
        if self._event is None:
            self._event = torch.cuda.Event()
        self._event.record()


class StepContext:
    """Passed to every part.  Device tensors are int32.

    ``token_ids`` [T], ``positions`` [T], ``want_rows`` [wanted], ``seq_slots`` [n] (state slot of
    each request), ``reset_slots`` [n] (the same for a request that starts in this step, else -1),
    ``q_starts`` [n+1], ``past_lens`` [n]; per paged group ``block_tables[g]``
    [n, pages] (units of the pool: page + 1; -1 = none, which reads the null page) and ``slots[g]``
    [T]; ``host`` holds the same as Python lists/arrays.
    ``plan(planner)`` gives the tables a part asked for through its ``planner()``."""

    def __init__(self, host: HostBatch, compute_dtype: torch.dtype, device):
        self.host = host
        self.compute_dtype = compute_dtype
        self.device = device
        self.n_tokens = host.n_tokens
        self.n_seqs = host.n_seqs
        self.token_ids = self.positions = self.want_rows = None
        self.seq_slots = self.q_starts = self.past_lens = self.reset_slots = None
        # set by the model: every norm can add up a delta that comes as float32 partial sums
        self.partial_sums_ok = False
        self.block_tables: List[torch.Tensor] = []
        self.slots: List[torch.Tensor] = []
        self.fresh_pages: List[Optional[torch.Tensor]] = []  # per group: units just taken from the pool, or None
        self._plans: Dict[Hashable, SimpleNamespace] = {}
        # what a part computes once per forward pass and its siblings in other layers use again
        # (keyed by whatever identifies it); emptied when a forward pass starts
        self.memo: Dict[Hashable, object] = {}

    def plan(self, planner) -> SimpleNamespace:
        try:
            return self._plans[planner.key]
        except KeyError:
            raise KeyError(f"no plan for {planner.key!r}: the part's planner() was not collected "
                           f"when the model was built") from None


def build_context(entries: Sequence[StepEntry], manager: CacheManager, planners: Sequence, staging: PinnedStaging,
                  compute_dtype: torch.dtype, device, pad: Optional[dict] = None,
                  into: Optional[torch.Tensor] = None, host: Optional[HostBatch] = None):
    """Tables of one step.  The entries' pages must have been reserved already.

    ``pad`` fixes the sizes of everything whose size depends on the requests' lengths (for a
    step that a captured graph replays): ``pad["pages"]`` = width of the block tables,
    ``pad[planner.key]`` = what that planner's ``graph_bucket`` returned.  ``host``: the host view
    of these very entries, if the caller has made it already.  Returns the context and the
    device buffer that holds all tables."""
    if host is None:
        host = HostBatch(entries, manager.page_size, compute_dtype)
    host.pad = pad
    ctx = StepContext(host, compute_dtype, device)
    pk = _Packer()
    i_ids = pk.add(host.token_ids.astype(np.int32))
    i_pos = pk.add(host.positions)
    i_want = pk.add(host.want_rows)
    i_slots = pk.add(np.asarray(host.seq_slots, dtype=np.int32))
    i_reset = pk.add(np.asarray(host.reset_slots, dtype=np.int32))
    i_qs = pk.add(np.asarray(host.q_starts, dtype=np.int32))
    i_past = pk.add(np.asarray(host.past_lens, dtype=np.int32))
    group_idx = []
    fresh_idx = []
    for g in range(len(manager.groups)):
        # pages just taken from the pool (as units: page + 1), for the kernel that zeroes them; a
        # replayed graph has room for one a request
        fresh = [p + 1 for e in entries for p in (getattr(e, "fresh", None) or [[]] * (g + 1))[g]]
        if pad is not None:
            if len(fresh) > len(entries):
                raise RuntimeError("more fresh pages than the captured graph has room for")
            fresh += [-1] * (len(entries) - len(fresh))
        fresh_idx.append(pk.add(np.asarray(fresh, dtype=np.int32)) if fresh else None)
        max_pages = max([len(e.cache.tables[g]) for e in entries] + [1])
        if pad is not None:
            if max_pages > pad["pages"]:
                raise RuntimeError("block tables are wider than the captured graph's")
            max_pages = pad["pages"]
        table = np.full((len(entries), max_pages), -1, dtype=np.int32)
        slot_map = np.full((host.n_tokens,), -1, dtype=np.int32)
        # the group's own geometry: a position lies in entry pos // tokens_per_entry, an entry in page
        # entry // entries_per_page
        per_entry, ps = manager.tokens_per_entry[g], manager.entries_per_page[g]
        for s, e in enumerate(entries):
            # page ids become units of the pool: unit 0 is the null page, page p is unit p + 1
            pages = np.asarray(e.cache.tables[g], dtype=np.int32)
            pages = np.where(pages >= 0, pages + 1, -1)
            table[s, :pages.size] = pages
            entry = host.positions[host.q_starts[s]:host.q_starts[s + 1]] // per_entry
            page_of = pages[entry // ps]
            slot_map[host.q_starts[s]:host.q_starts[s + 1]] = np.where(page_of >= 0, page_of * ps + entry % ps, -1)
        group_idx.append((pk.add(table), pk.add(slot_map)))
    plan_idx = []
    for planner in planners:
        made = planner.plan(host)
        arrays = {k: pk.add(v) for k, v in made.items() if isinstance(v, np.ndarray)}
        scalars = {k: v for k, v in made.items() if not isinstance(v, np.ndarray)}
        plan_idx.append((planner.key, arrays, scalars))
    dev = pk.upload(staging, device, into)
    ctx.token_ids, ctx.positions, ctx.want_rows = dev[i_ids], dev[i_pos], dev[i_want]
    ctx.seq_slots, ctx.q_starts, ctx.past_lens = dev[i_slots], dev[i_qs], dev[i_past]
    ctx.reset_slots = dev[i_reset]
    for it, isl in group_idx:
        ctx.block_tables.append(dev[it])
        ctx.slots.append(dev[isl])
    ctx.fresh_pages = [None if i is None else dev[i] for i in fresh_idx]
    for key, arrays, scalars in plan_idx:
        ctx._plans[key] = SimpleNamespace(**{k: dev[i] for k, i in arrays.items()}, **scalars)
    base = dev[0]._base if dev and dev[0]._base is not None else (dev[0] if dev else None)
    return ctx, base
