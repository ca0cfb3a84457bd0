"""Grouped-query attention over the paged cache."""

from __future__ import annotations

import math
from typing import Dict, Optional

import numpy as np
import torch

from .. import ops
from ..cache.manager import PagedNeed
from ..ops.functions import ATTN_ITEM_INTS, ATTN_MERGE_INTS
from ..ops.functions import GEMM_MFMA_SKINNY_BEST_M
from .base import Mixer, Norm, ParamDecl, Part, PositionEncoding, register_part
from .linear import Linear


class AttentionPlanner:
    """Cuts a step into the work items of the attention kernels (host side, once per step for all
    layers with the same geometry).

    A request's portion of n tokens at past length p becomes tiles of query tokens; a tile reads
    the keys from the start of its window to its last token.  A portion of at most
    ``small_tokens`` tokens is one *small* item.  A small item that reads more than ``split_keys``
    keys (decoding against a long context) is split over the keys into several items and merged
    afterwards in the order of the splits: 256 keys an item for the float32-arithmetic kernel (128
    or 64 by the same rule as below); for
    the matrix-core kernel, which gives every 128 keys to a wave of the item's workgroup and
    combines those inside, 1,024 keys, or 512, 256 or 128 while that leaves the step with at most
    as many workgroups as the device has compute units (every wave still sums the same 128 keys;
    only where their sums meet changes).  Longer portions are cut into *large* tiles of ``large_tokens``; how they are
    cut depends on the portion alone, never on what else is in the batch.  The item table lists
    the small items first.

    Two geometries exist: the matrix-core kernel (bfloat16, head size a multiple of 16, page size
    a multiple of 4) and the float32-arithmetic kernel for everything else; which one a step
    uses follows from the step's dtype and page size."""

    # Keys above which a large tile is given four waves that split its keys.  Off: idle waves in
    # the four-wave workgroups cost more than the balance gains.
    long_keys: Optional[int] = None
    # Compute units to fill with the workgroups of small items; None: those of the device.
    compute_units: Optional[int] = None

    def __init__(self, n_heads: int, n_kv: int, head_dim: int, window: Optional[int]):
        self.n_heads, self.n_kv, self.head_dim, self.window = n_heads, n_kv, head_dim, window
        self.key = ("attention", n_heads, n_kv, head_dim, window)
        self._geometry = {}

    def geometry(self, mfma: bool):
        """(small_tokens, large_tokens, split_keys) of a kernel family."""
        if mfma not in self._geometry:
            group = self.n_heads // self.n_kv
            if mfma:
                small = max(1, ops.attention_mfma_rows(self.head_dim, False) // min(group, 16))
                rows = ops.attention_mfma_rows(self.head_dim, True)
                large = max(1, rows // min(group, rows))
                # at most 1,024 keys (eight waves of 128) an item
                self._geometry[mfma] = (small, large, 128 * min(8, ops.attention_mfma_max_waves(self.head_dim)))
            else:
                t = ops.attention_tile_tokens(self.n_heads, self.n_kv)
                self._geometry[mfma] = (t, t, 256)
        return self._geometry[mfma]

    def uses_mfma(self, compute_dtype, page_size: int) -> bool:
        return (compute_dtype == torch.bfloat16 and self.head_dim % 16 == 0 and self.head_dim <= 256
                and page_size % 4 == 0)

    def _waves_for(self, keys: int, max_waves: int) -> int:
        """Waves of a workgroup for an item of ``keys`` keys: one per 128 keys, a power of two."""
        need = max(1, -(-keys // 128))
        w = 1
        while w < need and w < max_waves:
            w *= 2
        return min(w, max_waves)

    def _small_keys(self, host, small_tokens):
        """Keys that each small portion of the step reads."""
        keys = []
        for s in range(host.n_seqs):
            n, p = host.q_lens[s], host.past_lens[s]
            if n <= small_tokens:
                keys.append(p + n - (max(0, p - self.window + 1) if self.window else 0))
        return keys

    def split_keys(self, host, mfma: bool) -> int:
        """Keys per small item in this step.  A workgroup draws only so much from memory, so a step
        with few requests is faster with more, shorter items although they cost a merge, and a full
        device keeps the long ones."""
        small_tokens, _, longest = self.geometry(mfma)
        units = self.compute_units if self.compute_units is not None else ops.compute_units()
        keys = self._small_keys(host, small_tokens)
        group = self.n_heads // self.n_kv
        # the float32-arithmetic kernel takes 32 keys a pass and up to 16 heads of a group a workgroup:
        # its items shorten to 64 keys (two passes) while compute units are idle
        rows, shortest, room = (ops.attention_mfma_rows(self.head_dim, False), 128, 1) if mfma else (16, 64, 2)
        per_item = self.n_kv * -(-group // min(group, rows))  # workgroups of one item
        split = longest
        if mfma and keys and len(keys) <= self.whole_requests and max(keys) <= longest:
            # one or two requests whose keys fit one item: the item stays whole and the step has no
            # merge at all; the waves of its workgroup deal the keys and combine through LDS
            return longest
        # halved while the halves' workgroups still number at most the compute units: beyond that a
        # split only adds a merge.  The float32-arithmetic kernel's workgroups are slower and several
        # share a unit: twice the units.
        # (the matrix-core kernel: up to exactly one workgroup a unit)
        most_groups = units * room + (1 if mfma else 0)
        while split > shortest and sum(-(-k // (split // 2)) for k in keys) * per_item < most_groups:
            split //= 2
        if self.fine_items and mfma and keys and split > shortest:
            # between that length and its half: the shortest multiple of 32 whose workgroups still number at most the units
            lo, hi = 0, (split - split // 2) // 32 - 1
            while lo < hi:
                mid = (lo + hi + 1) // 2
                if sum(-(-k // (split - 32 * mid)) for k in keys) * per_item < most_groups:
                    lo = mid
                else:
                    hi = mid - 1
            split -= 32 * lo
        # requests that fit one item each need no merge at all while they stay whole: cutting them in
        # two is not worth one, in three or more it is
        if keys and split < longest and max(keys) <= longest and -(-max(keys) // split) <= 2:
            return longest
        # Items of the matrix-core kernel may be longer: the waves of a workgroup deal an item's keys
        # among themselves, and an item more for a request costs the work before the walk again and
        # a merge.  Where the requests alone give every compute unit a workgroup they stay whole,
        # however long.  Fewer requests take the longest items of which the full ones still number the
        # units; fewer workgroups than units lose.
        if self.long_items and mfma and keys and split == longest and units > 0 and max(keys) > longest:
            long = longest
            while long < max(keys):
                long *= 2
            # (no item longer than the keys a unit gets when they are dealt evenly, as a power of two:
            # one request of 100,000 keys among 63 short ones is cut, or its workgroups would run long
            # after the others)
            even = sum(keys) * per_item / units
            most = longest
            while most < even:
                most *= 2
            long = min(long, most)
            if len(keys) * per_item < units:
                while long > longest and sum(max(1, k // long) for k in keys) * per_item < units:
                    long //= 2
            split = long
        # Two cases in which shorter items are faster (measured at 28/4 and 40/8 heads of 128):
        # * more workgroups than units, in rounds of which the last is mostly empty: the items shorten
        #   as far as the same number of rounds still holds all their workgroups.  Items of less than a
        #   quarter of the length (the one key by which a request has passed a multiple) do not count
        #   as workgroups here: they are over at once.
        # * long items (twice the usual longest and more) whose workgroups leave the units half empty: a
        #   unit holds two such workgroups, so the items shorten as far as two a unit allow.  Not where
        #   no request is cut at all: whole requests that fill the units read at the memory's rate as
        #   they are, and cut in two they only gain a merge.
        # Both in steps of a 64th of the length (at least 32 keys) and to no less than half of it.
        if self.fill_rounds and mfma and keys and units > 0:
            def groups_of(length, least=0):
                return sum(k // length + (1 if k % length > least else 0) for k in keys) * per_item
            everyone, large_ones = groups_of(split), groups_of(split, split // 4)
            rounds = -(-large_ones // units)
            room_for = 0
            if large_ones > units and large_ones * 10 < rounds * units * 9:
                room_for = rounds * units
            elif split >= 2 * longest and everyone * 2 <= units * 3 and max(keys) > split:
                room_for = 2 * units
            if room_for:
                step = max(32, split // 64 // 32 * 32)
                # the shortest length on the grid whose workgroups still fit (their number only grows as
                # the items shorten): by halving the range
                lo, hi = 0, (split - split // 2) // step  # steps below `split`: lo fits, hi is the most
                while lo < hi:
                    mid = (lo + hi + 1) // 2
                    if groups_of(split - mid * step) <= room_for:
                        lo = mid
                    else:
                        hi = mid - 1
                shorter = split - lo * step
                if groups_of(shorter, shorter // 4) > large_ones:  # (shorter items that are no more items gain nothing)
                    split = shorter
        return split

    long_items = True  # items beyond the longest of `geometry` where they still fill the device
    # Steps of up to so many requests keep items that fit the longest whole (no merge launch).  0:
    # never, which is faster: the one-wave item asks for all its blocks of keys at once, a wave of the
    # many-wave workgroup for two at a time.
    whole_requests = 0
    # items shorten so that the last round of their workgroups is a full one (see split_keys)
    fill_rounds = True
    # between a power of two and its half, the shortest items whose workgroups still number at most the units
    fine_items = True

    @staticmethod
    def _items_of(keys: int, split_keys: int, longest: int) -> int:
        """Items that the ``keys`` keys of a small portion are cut into: runs of ``split_keys``."""
        return max(1, -(-keys // split_keys))

    def graph_bucket(self, host):
        """What a captured graph of this step's shape must fix: the number of (small) work items,
        the waves per item and the keys per item; None if the step has portions that do not fit
        small items."""
        mfma = self.uses_mfma(host.compute_dtype, host.page_size)
        small_tokens = self.geometry(mfma)[0]
        split_keys = self.split_keys(host, mfma)
        most = self.geometry(mfma)[2]
        n, longest = 0, 1
        for s in range(host.n_seqs):
            if host.q_lens[s] > small_tokens:
                return None
            first_key = max(0, host.past_lens[s] - self.window + 1) if self.window else 0
            keys = host.past_lens[s] + host.q_lens[s] - first_key
            mine = self._items_of(keys, split_keys, most)
            longest = max(longest, keys - (mine - 1) * split_keys)  # (the last item; the others have split_keys, if any)
            if mine > 1:
                longest = max(longest, split_keys)
            n += mine
        if mfma:
            # items: a multiple of the number of requests and of a quarter of what gives every unit a
            # workgroup, so that one graph serves a batch while its requests grow: their items grow
            # longer, not more (the captured graph pads with empty items, whose workgroups leave at
            # once).  The length of the items is data of the step, not of the graph.
            units = self.compute_units if self.compute_units is not None else ops.compute_units()
            group = self.n_heads // self.n_kv
            per_item = self.n_kv * -(-group // min(group, ops.attention_mfma_rows(self.head_dim, False)))
            step = max(host.n_seqs, units // per_item // 4, 1)
            return (-(-n // step) * step,
                    self._waves_for(longest, ops.attention_mfma_max_waves(self.head_dim)), 0)
        step = host.n_seqs * max(1, 1024 // split_keys)
        return (-(-n // step) * step, 1, split_keys)

    def plan(self, host) -> Dict[str, object]:
        mfma = self.uses_mfma(host.compute_dtype, host.page_size)
        small_tokens, large_tokens, most = self.geometry(mfma)
        padded = getattr(host, "pad", None) is not None
        split_keys = self.split_keys(host, mfma)
        small, merges = [], []
        large_runs = []  # per long portion: its tiles as rows of an array (a prompt of thousands of tokens has hundreds)
        n_partial = 0
        for s in range(host.n_seqs):
            n, p, row0 = host.q_lens[s], host.past_lens[s], host.q_starts[s]
            first_key = max(0, p - self.window + 1) if self.window else 0
            total = p + n
            n_splits = self._items_of(total - first_key, split_keys, most) if split_keys is not None else 1
            if n <= small_tokens and n_splits > 1:
                base = n_partial
                for i in range(n_splits):
                    kb = first_key + i * split_keys
                    small.append((s, row0, n, p, kb, total if i == n_splits - 1 else kb + split_keys, base + i * n, 0))
                for t in range(n):
                    merges.append((row0 + t, base + t, n_splits, n))
                n_partial += n_splits * n
            elif n <= small_tokens:
                small.append((s, row0, n, p, first_key, total, -1, 0))
            else:
                # (the short tile that a long portion may end with stays with the portion's other tiles:
                # as a small item it would walk all the portion's keys in one workgroup a kv head, alone
                # on the device, while as the last of a group of four it shares their blocks of keys)
                t0 = np.arange(0, n, large_tokens, dtype=np.int64)
                run = np.empty((t0.shape[0], ATTN_ITEM_INTS), dtype=np.int64)
                pos0 = p + t0
                run[:, 0] = s
                run[:, 1] = row0 + t0
                run[:, 2] = np.minimum(large_tokens, n - t0)
                run[:, 3] = pos0
                run[:, 4] = np.maximum(0, pos0 - self.window + 1) if self.window else 0
                run[:, 5] = pos0 + run[:, 2]
                run[:, 6] = -1
                run[:, 7] = 0
                large_runs.append(run)
        large = np.concatenate(large_runs) if large_runs else np.zeros((0, ATTN_ITEM_INTS), dtype=np.int64)
        waves = 1
        if mfma and small:
            waves = self._waves_for(max(it[5] - it[4] for it in small), ops.attention_mfma_max_waves(self.head_dim))
        if padded:
            # a captured graph launches fixed grids: pad with items and merges that do nothing
            n_items, waves, _ = host.pad[self.key]
            if len(large) or len(small) > n_items:
                raise RuntimeError("attention plan does not fit the captured graph")
            small += [(0, 0, 0, 0, 0, 0, -1, 0)] * (n_items - len(small))
            if n_items > host.n_seqs:
                # the graph has room for items that share a request's keys: it merges every row
                # (rows that need none get an empty merge)
                merged = {m[0] for m in merges}
                merges += [(row, 0, 0, 0) for row in range(host.n_tokens) if row not in merged]
                n_partial = n_items * small_tokens
        # consecutive large tiles of one request, four at a time, for the kernel that shares the
        # keys of a block among four waves
        groups = np.zeros((0, 2), dtype=np.int64)
        if mfma and large_runs:
            firsts, counts, at = [], [], 0
            for run in large_runs:
                f = np.arange(0, run.shape[0], 4, dtype=np.int64)
                firsts.append(at + f)
                counts.append(np.minimum(4, run.shape[0] - f))
                at += run.shape[0]
            firsts, counts = np.concatenate(firsts), np.concatenate(counts)
            # by the number of keys a group goes through, ascending: the kernel starts its workgroups
            # from the back of this list, the longest first (with several requests in a step the
            # order of the requests would otherwise decide)
            order = np.argsort(large[firsts + counts - 1, 5] - large[firsts, 4], kind="stable")
            groups = np.stack([firsts[order], counts[order]], axis=1)
        n_long = 0
        if mfma and self.long_keys is not None:
            # large tiles that read more than ``long_keys`` keys go to workgroups of four waves
            is_long = large[:, 5] - large[:, 4] > self.long_keys
            large = np.concatenate([large[~is_long], large[is_long]])
            n_long = int(is_long.sum())
        small_items = np.asarray(small, dtype=np.int64).reshape(-1, ATTN_ITEM_INTS)
        return {
            "items": np.concatenate([small_items, large]).astype(np.int32),
            "merges": np.asarray(merges, dtype=np.int32).reshape(-1, ATTN_MERGE_INTS),
            "groups": groups.astype(np.int32), "n_groups": len(groups),
            "n_small": len(small), "n_large": len(large) - n_long, "n_long": n_long, "n_merges": len(merges),
            "n_partial": n_partial, "mfma": mfma, "waves": waves,
            "single": all(host.q_lens[s] == 1 for s in range(host.n_seqs)),  # one token a request
        }


@register_part("mixer", "gqa_attention")
class GQAttention(Mixer):
    """q/k/v projections (one matrix, optional bias), optional norms of every q and k head,
    position encoding, causal attention with kv head = q head // (heads / kv heads) and scale
    1/sqrt(head_dim), output projection without bias (src/model/model.cpp:110-129,
    src/model/nn.cpp:151-226).  ``window`` = number of latest positions a query reads (None: all).

    What happens between the projection and attention, in this order: bias, ``q_norm`` / ``k_norm``
    (a norm as wide as a head, applied to every head through ``Norm.plain``; None: none), the
    position encoding's ``rotate``, the write of k and v into the cache.  The mixer owns all of it;
    the encoding only rotates.  Where nothing stands between the projection and a rotation that
    the encoding can describe by a table of cosines and sines (``rotation_table``), the mixer's own
    kernels do several of these steps at once: for steps of one token a request the attention
    kernel itself finishes the projection's partial sums (bias, rotation, cache write); for up to 16
    rows the projection's epilogue does; for 17 to 128 rows the kernel that writes the cache adds
    the partial sums up.  With head norms, or an encoding without a table, the steps run one after
    the other (projection, bias, norms, ``rotate``, cache write), which every combination can take."""

    share_keys = True  # long portions: four tiles of a request share each block of keys through LDS
    # steps of one token a request: the attention kernel adds up the q/k/v product's partial sums,
    # rotates and writes the cache itself (one launch fewer a layer)
    finish_qkv_in_attention = True

    @property
    def graph_safe(self) -> bool:
        """forward reads the step only through device tables; its sub-parts must too."""
        return all(p.graph_safe for p in self.sub_parts().values())

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, qkv_bias: bool,
                 position: PositionEncoding, window: Optional[int] = None, q_norm: Optional[Norm] = None,
                 k_norm: Optional[Norm] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: heads {n_heads} must be a multiple of kv heads {n_kv_heads}")
        if head_dim > 256:
            raise ValueError(f"attention: head_dim {head_dim} is larger than the kernels take (256)")
        self.hidden_size, self.n_heads, self.n_kv, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.window = window
        self.position = position
        self.q_norm, self.k_norm = q_norm, k_norm
        self.q_dim, self.kv_dim = n_heads * head_dim, n_kv_heads * head_dim
        self.qkv = Linear(hidden_size, self.q_dim + 2 * self.kv_dim, bias=qkv_bias)
        self.o = Linear(self.q_dim, hidden_size)
        self.scale = 1.0 / math.sqrt(head_dim)
        self._planner: Optional[AttentionPlanner] = None

    def sub_parts(self) -> Dict[str, Part]:
        parts: Dict[str, Part] = {"position": self.position}
        if self.q_norm is not None:
            parts["q_norm"] = self.q_norm
        if self.k_norm is not None:
            parts["k_norm"] = self.k_norm
        return parts

    # parameters -------------------------------------------------------------------------
    def param_decls(self) -> Dict[str, ParamDecl]:
        decls = {"qkv_weight": ParamDecl((self.q_dim + 2 * self.kv_dim, self.hidden_size)),
                 "o_weight": ParamDecl((self.hidden_size, self.q_dim))}
        if self.qkv.has_bias:
            decls["qkv_bias"] = ParamDecl((self.q_dim + 2 * self.kv_dim,), "vector", "bias")
        return decls

    qkv_weight = property(lambda s: s.qkv.weight, lambda s, t: setattr(s.qkv, "weight", t))
    qkv_bias = property(lambda s: s.qkv.bias, lambda s, t: setattr(s.qkv, "bias", t))
    o_weight = property(lambda s: s.o.weight, lambda s, t: setattr(s.o, "weight", t))

    def prepare(self, device, compute_dtype) -> None:
        copies = bool(self.options.get("weight_copies", True))
        self.o.prepare(copies)
        self.qkv.prepare(copies)  # (read by the product of 17 to 64 rows; the few-rows product with the rotation reads rows)

    def release_optional_memory(self) -> int:
        return self.qkv.drop_copy() + self.o.drop_copy()

    # cache and plan ---------------------------------------------------------------------
    def cache_need(self) -> PagedNeed:
        return PagedNeed(self.n_kv, self.head_dim, self.window)

    def planner(self) -> AttentionPlanner:
        if self._planner is None:
            self._planner = AttentionPlanner(self.n_heads, self.n_kv, self.head_dim, self.window)
        return self._planner

    # compute ----------------------------------------------------------------------------
    def _fused_table(self, ctx) -> Optional[torch.Tensor]:
        """The rotation as a table, if the mixer's fused kernels may stand for bias + rotate + write:
        nothing between the projection and the rotation, and an encoding that is such a rotation
        (or none at all: then the kernels only add the bias and write)."""
        if self.q_norm is not None or self.k_norm is not None or self.head_dim % 8:
            return None
        return self.position.rotation_table(self.head_dim, ctx)

    def _from_sums(self, x: torch.Tensor, ctx, cache, plan, table) -> Optional[torch.Tensor]:
        """Attention of a step of one token a request straight from the q/k/v product's partial sums
        (None: not such a step, or the kernels do not take the sizes)."""
        if not (self.finish_qkv_in_attention and table is not None and cache.writes and plan.mfma and plan.single
                and plan.n_small and not plan.n_large and not plan.n_long and x.dtype == torch.bfloat16
                and ops.attention_mfma_qkv_ok(self.head_dim, cache.page_size)):
            return None
        sums = self.qkv.partial_sums(x, few_rows=True)
        if sums is None:
            return None
        out = torch.empty((x.shape[0], self.q_dim), dtype=x.dtype, device=x.device)
        partials = None
        if plan.n_partial:
            partials = torch.empty((plan.n_partial * self.n_heads * (self.head_dim + 2),), dtype=torch.float32,
                                   device=x.device)
        ops.attention_mfma_qkv(sums, self.qkv.bias, table, cache.slots, cache.k_pool, cache.v_pool,
                               cache.block_tables, plan.items, plan.n_small, out, partials, self.n_heads, self.n_kv,
                               self.head_dim, self.window, self.scale, waves=plan.waves)
        if plan.n_merges:
            ops.attention_merge(partials, plan.merges, plan.n_merges, out, self.n_heads, self.head_dim)
        return out

    def _project_rotate_store(self, x: torch.Tensor, ctx, cache, table) -> torch.Tensor:
        """q/k/v [T, (heads + 2 kv heads) head_dim] of which attention reads the q columns: projected,
        with the bias, the head norms and the rotation applied, and k and v written into the cache
        (unless this call only reads another call's cache)."""
        nh, nkv, hd = self.n_heads, self.n_kv, self.head_dim
        store = dict(slots=cache.slots, k_pool=cache.k_pool, v_pool=cache.v_pool,
                     page_size=cache.page_size) if cache.writes else {}
        bias = self.qkv.bias
        if table is not None:
            if x.dtype == torch.bfloat16 and 0 < x.shape[0] <= GEMM_MFMA_SKINNY_BEST_M and x.shape[1] % 8 == 0 and hd % 16 == 0:
                # a few rows of a step that is not one token a request: the projection's own epilogue
                # adds the bias, rotates and stores
                return ops.gemm_mfma_skinny_rope(x, self.qkv.weight, bias, ctx.positions, nh, nkv, hd, None,
                                                 cos_sin=table, **store)
            sums = self.qkv.partial_sums(x)
            if sums is not None:
                # 17 to 128 rows: the engine's product in slices of K, added up by the kernel that rotates
                qkv = torch.empty(sums.shape[1:], dtype=ctx.compute_dtype, device=x.device)
                return ops.rope_kv_write(qkv, ctx.positions, nh, nkv, hd, None, bias=bias, cos_sin=table,
                                         parts=sums, **store)
        qkv = self.qkv(x, skip_bias=True)
        if table is not None:
            return ops.rope_kv_write(qkv, ctx.positions, nh, nkv, hd, None, bias=bias, cos_sin=table, **store)
        # one step after the other
        plain_write = not self.position.rotates and self.q_norm is None and self.k_norm is None
        if bias is not None and not plain_write:
            ops.bias_add(qkv, bias)
            bias = None
        if self.q_norm is not None:
            q = qkv[:, :self.q_dim]
            self.q_norm.plain(q, out=q)
        if self.k_norm is not None:
            k = qkv[:, self.q_dim:self.q_dim + self.kv_dim]
            self.k_norm.plain(k, out=k)
        if self.position.rotates:
            self.position.rotate(qkv, nh, nkv, hd, ctx)
        if store or bias is not None:
            ops.rope_kv_write(qkv, ctx.positions, nh, nkv, hd, None, bias=bias, **store)  # (no rotation: bias, write)
        return qkv

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        plan = ctx.plan(self.planner())
        table = self._fused_table(ctx)
        out = self._from_sums(x, ctx, cache, plan, table)
        if out is not None:
            return self.o.for_residual(out, ctx)
        qkv = self._project_rotate_store(x, ctx, cache, table)
        t = x.shape[0]
        out = torch.empty((t, self.q_dim), dtype=x.dtype, device=x.device)
        partials = None
        if plan.n_partial:
            partials = torch.empty((plan.n_partial * self.n_heads * (self.head_dim + 2),), dtype=torch.float32,
                                   device=x.device)
        args = (partials, self.n_heads, self.n_kv, self.head_dim, self.window, self.scale, t)
        if plan.mfma:
            if plan.n_small:
                ops.attention_mfma(qkv, qkv.shape[1], cache.k_pool, cache.v_pool, cache.block_tables, plan.items,
                                   plan.n_small, out, *args, large=False, waves=plan.waves)
            if plan.n_large and not plan.n_long and self.share_keys and ops.attention_mfma_lds_ok(self.head_dim,
                                                                                                   cache.page_size):
                ops.attention_mfma_lds(qkv, qkv.shape[1], cache.k_pool, cache.v_pool, cache.block_tables,
                                       plan.items[plan.n_small:], plan.groups, plan.n_groups, out, self.n_heads,
                                       self.n_kv, self.head_dim, self.window, self.scale, t)
            elif plan.n_large:
                ops.attention_mfma(qkv, qkv.shape[1], cache.k_pool, cache.v_pool, cache.block_tables,
                                   plan.items[plan.n_small:], plan.n_large, out, *args, large=True)
            if plan.n_long:
                ops.attention_mfma(qkv, qkv.shape[1], cache.k_pool, cache.v_pool, cache.block_tables,
                                   plan.items[plan.n_small + plan.n_large:], plan.n_long, out, *args, large=True,
                                   waves=4)
        else:
            ops.attention_scalar(qkv, qkv.shape[1], cache.k_pool, cache.v_pool, cache.block_tables, plan.items,
                                 plan.n_small + plan.n_large, out, *args)
        if plan.n_merges:
            ops.attention_merge(partials, plan.merges, plan.n_merges, out, self.n_heads, self.head_dim)
        return self.o.for_residual(out, ctx)
