"""The model on the device and the step function.

``Model`` owns the parts with their weights.  ``Runner`` joins a model with a cache (manager +
storage) and offers ``step``: run the given tokens of the given requests as one batch, from the
cache that earlier steps left, and return the logits at the wanted places.
"""

from __future__ import annotations

from pathlib import Path
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from ..cache.allocator import OutOfPages
from ..cache.manager import CacheManager
from ..cache.needs import CacheNeed
from ..cache.storage import CacheLayout, CacheStorage
from ..config.base import ModelConfig, read_config_json
from ..models.registry import build_model_spec, parse_config
from ..models.spec import ModelSpec
from ..parts.base import HiddenState, prepare_parts
from ..weights.loader import fill_parts, load_weights
from ..weights.random_init import random_tensor, expected_tensors
from .context import PinnedStaging, StepContext, StepEntry, build_context, filler_entry

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine runs in bfloat16 or float32, not {dtype}")
        return dtype
    try:
        return _DTYPES[str(dtype)]
    except KeyError:
        raise ValueError(f"unknown dtype '{dtype}' (bfloat16 or float32)") from None


def _require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("the engine needs a GPU: there is no CPU path")
    ops.load()  # fails loudly when the kernel library is missing
    return device


class Model:
    def __init__(self, spec: ModelSpec, dtype, device):
        self.spec = spec
        self.config = spec.config
        self.dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        self.weight_bytes = 0
        # caches: one per call of the schedule that keeps one
        self.call_cache: List[int] = []
        needs: Dict[int, object] = {}
        for i, call in enumerate(spec.schedule):
            if not 0 <= call.layer < len(spec.layers):
                raise ValueError(f"schedule entry {i} names layer {call.layer}, which does not exist")
            if call.cache_of is None:
                self.call_cache.append(i)
                need = spec.layers[call.layer].mixer.cache_need()
                if need is not None:
                    needs[i] = need
            else:
                if not 0 <= call.cache_of < i or spec.schedule[call.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {i}: cache_of must name an earlier call that keeps a cache")
                self.call_cache.append(call.cache_of)
        # per-token needs that compare equal share a pool of pages (a group); a per-request need
        # gets slots of its own.  What the memory looks like is the need's business.
        groups: List[CacheNeed] = []
        group_caches: List[List[int]] = []
        states: Dict[int, CacheNeed] = {}
        for cid, need in needs.items():
            per_token = getattr(need, "per_token", None)
            if not isinstance(per_token, bool) or not callable(getattr(need, "allocate", None)):
                raise TypeError(f"cache_need() of call {cid} returned {type(need).__name__}, which is no cache need "
                                f"(per_token, allocate, view)")
            if per_token:
                if need not in groups:
                    groups.append(need)
                    group_caches.append([])
                group_caches[groups.index(need)].append(cid)
            else:
                states[cid] = need
        self.cache_layout = CacheLayout(groups, group_caches, states)
        self.cached_calls = set(needs)
        # planners of all mixers, one per distinct key
        self.planners = []
        seen = set()
        for block in spec.layers:
            planner = block.mixer.planner()
            if planner is not None and planner.key not in seen:
                seen.add(planner.key)
                self.planners.append(planner)

    # ---------------------------------------------------------------- construction
    @classmethod
    def from_pretrained(cls, model_dir, dtype="bfloat16", device="cuda:0", weight_copies: bool = True) -> "Model":
        """``weight_copies=False``: no second, fragment-ordered copy of the large matrices (half
        the memory; decode steps then read rows and are some 8 % slower)."""
        device = _require_gpu(device)
        config = parse_config(read_config_json(model_dir))
        model = cls(build_model_spec(config), dtype, device)
        model.weight_bytes = load_weights(Path(model_dir), model.spec.bindings, model.dtype, device,
                                          model.spec.ignore_unexpected)
        model._prepare(weight_copies)
        return model

    @classmethod
    def from_random(cls, config: ModelConfig, seed: int = 0, dtype="bfloat16", device="cuda:0",
                    weight_copies: bool = True) -> "Model":
        """Random weights without a folder, drawn on the device (gigabytes in a fraction of a
        second): the very values that ``write_random_model`` writes for this configuration and
        seed (the generator is a function of seed, tensor name and element index)."""
        device = _require_gpu(device)
        model = cls(build_model_spec(config), dtype, device)
        specs = expected_tensors(model.spec.bindings)
        model.weight_bytes = fill_parts(
            model.spec.bindings, lambda name: random_tensor(specs[name], seed, torch.float32, device=device),
            model.dtype, device)
        model._prepare(weight_copies)
        return model

    def _prepare(self, weight_copies: bool = True) -> None:
        self.options = {"weight_copies": bool(weight_copies)}
        seen: set = set()
        for part in self.spec.all_parts():
            prepare_parts(part, self.device, self.dtype, self.options, seen)
        self.partial_sums_ok = all(norm.adds_partial_sums for norm in self.spec.stream_norms())

    # ---------------------------------------------------------------- cache
    def make_cache(self, page_size: int, num_pages: int, max_requests: int):
        """The cache's host and device side.  The second copies of the large weights were made before
        the cache's size was known: if the pools do not fit beside them, the copies go (decode steps
        then read rows, some 8 % slower) and the pools are asked for once more."""
        manager = CacheManager(self.cache_layout.paged_groups, page_size, num_pages, max_requests)
        try:
            storage = CacheStorage(self.cache_layout, manager, self.device, self.dtype)
        except torch.cuda.OutOfMemoryError:
            freed = sum(part.release_optional_memory() for part in self.spec.all_parts())
            if not freed:
                raise
            torch.cuda.empty_cache()
            import warnings

            warnings.warn(f"the cache of {num_pages} pages did not fit beside the second copies of the large weights: "
                          f"{freed / 2 ** 30:.1f} GiB of copies dropped (as with weight_copies=False)")
            storage = CacheStorage(self.cache_layout, manager, self.device, self.dtype)
        return manager, storage

    def cache_bytes_per_token(self) -> int:
        return sum(need.bytes_per_token(self.dtype) * len(ids)
                   for need, ids in zip(self.cache_layout.paged_groups, self.cache_layout.group_caches))

    def pages_that_fit(self, page_size: int) -> int:
        """Pages of ``page_size`` tokens that the device's free memory holds beside what is loaded
        (nine tenths of it, less 2 GiB for a step's activations, graphs and workspaces), and no
        more than keep every layer's pools below 2^31 elements (pools beyond that can be asked for
        by their number of pages; none has been run)."""
        from ..cache.manager import pages_that_fit

        per_token = self.cache_bytes_per_token()
        if per_token <= 0:
            raise ValueError("the cache's needs do not say how many bytes a token takes: give the number of pages")
        free, _ = torch.cuda.mem_get_info(self.device)
        pages = pages_that_fit(free, per_token, page_size)
        itemsize = torch.empty((), dtype=self.dtype).element_size()
        per_layer = max(need.bytes_per_token(self.dtype) for need in self.cache_layout.paged_groups) // itemsize
        return max(1, min(pages, (2 ** 31 - 1) // max(1, per_layer * page_size)))

    # ---------------------------------------------------------------- compute
    def forward(self, ctx: StepContext, storage: CacheStorage) -> torch.Tensor:
        """float32 logits [wanted, vocab] for the step described by ``ctx``."""
        spec = self.spec
        ctx.partial_sums_ok = self.partial_sums_ok
        ctx.memo.clear()  # a captured graph must hold whatever the layers share: nothing is kept from an earlier pass
        storage.reset_states(ctx)  # requests that start in this step find their per-request memory zero
        storage.clear_fresh(ctx)   # and the pages taken from the pools for this step hold nothing of their last owner
        hidden = HiddenState(spec.embedding.forward(ctx.token_ids))
        for i, call in enumerate(spec.schedule):
            cid = self.call_cache[i]
            cache = storage.view(cid, ctx, writes=call.cache_of is None) if cid in self.cached_calls else None
            spec.layers[call.layer].forward(hidden, ctx, cache)
        if ctx.want_rows.shape[0] == 0:
            return torch.empty((0, spec.lm_head.vocab_size), dtype=torch.float32, device=self.device)
        normed = spec.final_norm.rows(hidden, ctx.want_rows, self.dtype)
        return spec.lm_head.forward(normed)


class Runner:
    """The step function over one model and one cache."""

    def __init__(self, model: Model, page_size: int = 16, num_pages: int = 2048, max_requests: int = 256,
                 use_graphs: bool = True, fill_rows=None):
        """``fill_rows``: optional policy ``tokens -> tokens`` of whoever made the runner: a step that
        is not replayed from a graph is filled up to that many rows with the tokens of a request that
        does not exist (``filler_entry``).  A caller that has the library's kernels timed for a few
        row counts passes ``padded_tokens``.  Only for models whose parts all read a step through its
        device tables (``graph_safe``): the filler's rows exist in those tables alone."""
        self.model = model
        self.fill_rows = fill_rows if all(p.graph_safe for p in model.spec.all_parts()) else None
        self.manager, self.storage = model.make_cache(page_size, num_pages, max_requests)
        self._staging = PinnedStaging()
        self.vocab_size = model.spec.embedding.vocab_size
        self.max_position = int(model.config.max_positions)  # 0: the architecture sets no limit
        self.steps = 0
        self.tokens = 0
        from .graphs import DecodeGraphs

        self.graphs = DecodeGraphs(self) if use_graphs else None

    def check(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise ValueError("step: empty batch")
        seen = set()
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"step: request {e.cache.request_id!r} brings no tokens")
            if e.cache.closed:
                raise ValueError(f"step: request {e.cache.request_id!r} is closed")
            if id(e.cache) in seen:
                raise ValueError(f"step: request {e.cache.request_id!r} appears twice in one step")
            seen.add(id(e.cache))
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= self.vocab_size:
                raise IndexError(f"step: token id {lo if lo < 0 else hi} of request {e.cache.request_id!r} "
                                 f"is outside the vocabulary [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= w < n:
                    raise IndexError(f"step: wanted place {w} is outside the {n} tokens of request "
                                     f"{e.cache.request_id!r}")
            if self.max_position and e.cache.length + n > self.max_position:
                raise ValueError(f"step: request {e.cache.request_id!r} would reach {e.cache.length + n} "
                                 f"positions, more than the model's limit of {self.max_position}")

    def step(self, entries: Sequence[StepEntry], keep: bool = True,
             feed: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run one batch.  Nothing is changed when the batch is refused (bad ids, no pages).
        ``keep=False`` allows the returned logits to live in a buffer that the next step
        overwrites (a caller that consumes them at once saves a copy).  ``feed``: an int32 device
        tensor with one token id per token of the batch, used instead of the entries' ids (which
        only stand in): ids that an earlier step has sampled and the host has not read yet."""
        self.check(entries)
        if feed is not None and (feed.dtype != torch.int32 or feed.ndim != 1 or
                                 feed.shape[0] != sum(len(e.tokens) for e in entries)):
            raise ValueError("step: feed must hold one int32 token id per token of the batch")
        if not self.manager.can_reserve((e.cache, len(e.tokens)) for e in entries):
            raise OutOfPages("step: the batch needs more pages than the pool has free")
        for e in entries:
            e.fresh = self.manager.reserve(e.cache, len(e.tokens))
        pad = self.graphs.shape_of(entries) if self.graphs is not None else None
        logits = self.graphs.step(entries, pad, feed) if pad is not None else None
        if logits is not None:
            if keep:
                logits = logits.clone()
        else:
            n_tokens = sum(len(e.tokens) for e in entries)
            batch = list(entries)
            extra = self.fill_rows(n_tokens) - n_tokens if self.fill_rows is not None else 0
            if extra > 0:
                batch.append(filler_entry(self.storage, extra))
            ctx, _ = build_context(batch, self.manager, self.model.planners, self._staging, self.model.dtype,
                                   self.model.device)
            if feed is not None:
                ctx.token_ids[:n_tokens].copy_(feed)
            logits = self.model.forward(ctx, self.storage)
        for e in entries:
            self.manager.commit(e.cache, len(e.tokens))
        self.steps += 1
        self.tokens += sum(len(e.tokens) for e in entries)
        return logits
