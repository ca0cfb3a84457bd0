"""Decode steps as replayed HIP graphs.

A decode step launches some ten kernels per layer, each a few microseconds long; queued one by
one from Python they cost more host time than GPU time.  A step whose every request brings one
token and wants its logits has a shape that depends only on the number of requests and, through
the width of the block tables (a power of two of pages) and the number of attention work items
and their waves, on coarsely rounded context lengths: how long the items are is data of a step,
so a batch keeps its graph while its requests grow, until the tables or the items double.  For
each such shape the whole forward is captured once into a graph that reads all its index tables
from one fixed device buffer; a later step of the same shape copies its tables there and replays
the graph.

The number of requests is rounded up as well (``padded_rows``): a batch that shrinks request by
request as they finish would otherwise want a new graph, some tens of milliseconds of capture,
at every size.  The rows that fill a batch up are requests of one token at position 0 whose
cache is the pools' spare page and the spare state slot; they cost a decode step nothing that
can be measured, no request reads what they write, and their logits are dropped.

A shape is captured when it comes for the third time (``capture_after``); until then its steps
run eagerly, which costs a few milliseconds of host time each where a capture costs thirty: the
shapes a batch passes through while its last requests end, one or two steps each, are not worth
a graph.
"""

from __future__ import annotations

import gc
import weakref
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .context import HostBatch, StepEntry, build_context, filler_entry

PAGE_BUCKET = 32  # block-table widths are at least this many pages (and powers of two)
CAPTURE_AFTER = 3  # a shape is captured the n-th time it is asked for (read when a runner is made)


def padded_rows(n: int) -> int:
    """Rows of the graph that serves a decode step of ``n`` requests: 1, 2, 4, 8, then multiples
    of 16 (a tile of rows in the products) up to 128, which is what the engine's own products
    take, above that of 32."""
    if n <= 8:
        return 1 << max(0, n - 1).bit_length()
    step = 16 if n <= 128 else 32
    return -(-n // step) * step


class DecodeGraphs:
    def __init__(self, runner, max_graphs: int = 64, capture_after: Optional[int] = None):
        # no cycle with the runner: a runner that is dropped must free its graphs and pinned
        # buffers then and there, not whenever the collector of cycles next runs (which may be
        # in the middle of another runner's capture, where freeing device memory is an error
        # that ends the process)
        self._runner = weakref.ref(runner)
        self.max_graphs = max_graphs
        self.capture_after = CAPTURE_AFTER if capture_after is None else capture_after
        self._asked: Dict[Tuple, int] = {}
        self._graphs: Dict[Tuple, Tuple[torch.cuda.CUDAGraph, torch.Tensor, torch.Tensor, torch.Tensor]] = {}
        model = runner.model
        # every part of the model: the embedding, the head and the final norm as well as the layers'
        self.enabled = (all(p.graph_safe for p in model.spec.all_parts())
                        and all(hasattr(p, "graph_bucket") for p in model.planners))
        self.replays = 0
        self.captures = 0
        self._host = None  # the host view that shape_of made, for the step that follows

    @property
    def runner(self):
        runner = self._runner()
        if runner is None:
            raise RuntimeError("the runner of these graphs no longer exists")
        return runner

    def filled_up(self, entries: Sequence[StepEntry]) -> List:
        """The entries and, behind them, the rows that pad the batch to a graph's size."""
        runner = self.runner
        filler = filler_entry(runner.storage, 1)
        filler.want = (0,)
        return list(entries) + [filler] * (padded_rows(len(entries)) - len(entries))

    def shape_of(self, entries: Sequence[StepEntry]) -> Optional[dict]:
        """The padded sizes of this step, or None if it is not a plain decode step."""
        if not self.enabled or not all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
            return None
        runner = self.runner
        entries = self.filled_up(entries)
        host = HostBatch(entries, runner.manager.page_size, runner.model.dtype)
        pages = max(len(t) for e in entries for t in e.cache.tables) if runner.manager.groups else 1
        # the width of the block tables: a power of two (at least PAGE_BUCKET pages), so that a batch whose
        # requests grow changes graphs once per doubling and not every few hundred tokens
        pad = {"pages": max(PAGE_BUCKET, 1 << (max(pages, 1) - 1).bit_length())}
        for planner in runner.model.planners:
            bucket = planner.graph_bucket(host)
            if bucket is None:
                return None
            pad[planner.key] = bucket
        self._host = host  # of the filled-up entries: the step that follows takes it instead of making it again
        return pad

    def step(self, entries: Sequence[StepEntry], pad: dict,
             feed: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run the (already reserved) decode step through its graph; returns the logits, which
        stay valid until the next step of the same shape, or None when the shape has no graph
        and is not due for one yet (the caller then runs the step eagerly).  ``feed`` (int32, on
        the device) replaces the token ids after the tables have been sent."""
        runner = self.runner
        n = len(entries)
        entries = self.filled_up(entries)
        host, self._host = self._host, None
        if host is not None and host.n_seqs != len(entries):
            host = None
        key = (len(entries),) + tuple(sorted((str(k), v) for k, v in pad.items()))
        hit = self._graphs.get(key)
        if hit is None:
            if len(self._asked) > 4096:
                self._asked.clear()
            asked = self._asked[key] = self._asked.get(key, 0) + 1
            if asked < self.capture_after:
                return None
            if len(self._graphs) >= self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
            # An eager run of the same shape first: it allocates what the graph must not, and warms
            # the library's kernel selection.  It runs on rows that belong to no request (the spare
            # page, the spare slot), so that the step itself is executed once and only once, by the
            # replay below: a part whose cache is a running state would otherwise advance it twice.
            warm = [filler_entry(runner.storage, 1) for _ in entries]
            for w in warm:
                w.want = (0,)
            warm_ctx, _ = build_context(warm, runner.manager, runner.model.planners, runner._staging,
                                        runner.model.dtype, runner.model.device, pad=pad)
            runner.model.forward(warm_ctx, runner.storage)
            torch.cuda.synchronize()
            del warm_ctx
            ctx, tables = build_context(entries, runner.manager, runner.model.planners, runner._staging,
                                        runner.model.dtype, runner.model.device, pad=pad, host=host)
            if feed is not None:
                ctx.token_ids[:n].copy_(feed)
            graph = torch.cuda.CUDAGraph()
            # Nothing may free device or pinned memory while the stream is captured.  Dead cycles
            # of Python objects that hold such memory (or other graphs) are therefore collected
            # now, and the collector stays off until the capture has ended.
            gc.collect()
            collector_was_on = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph):
                    logits = runner.model.forward(ctx, runner.storage)
            finally:
                if collector_was_on:
                    gc.enable()
            self._graphs[key] = (graph, tables, logits, ctx.token_ids)
            self.captures += 1
            graph.replay()  # the step itself
            return logits[:n]
        graph, tables, logits, token_ids = hit
        build_context(entries, runner.manager, runner.model.planners, runner._staging, runner.model.dtype,
                      runner.model.device, pad=pad, into=tables, host=host)
        if feed is not None:
            token_ids[:n].copy_(feed)
        graph.replay()
        self.replays += 1
        return logits[:n]
