"""The host side of attention: how a step is cut into work items (no GPU needed; the geometry
comes from host functions of the kernel library).

For random batches, both kernel families and with and without a window: every query sees each
key of its range exactly once over its items, rows whose keys are split have one partial slot per
split and one merge that names them in order, no slot is used twice, groups for the LDS kernel
are consecutive tiles of one request, and a request is cut the same way alone and in a batch."""

import random

import numpy as np
import pytest
import torch

from from_scratch_inference_engine_amd import ops
from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

try:  # the tile sizes are host functions of the kernel library (built at first use where hipcc exists)
    ops.load()
except ops.KernelLibraryMissing as e:  # pragma: no cover
    pytest.skip(f"no kernel library: {e}", allow_module_level=True)

SEQ, ROW, NQ, POS, KB, KE, PARTIAL = range(7)


class Host:
    def __init__(self, seqs, page_size, dtype):
        self.n_seqs = len(seqs)
        self.past_lens = [p for p, _ in seqs]
        self.q_lens = [n for _, n in seqs]
        self.q_starts = [0]
        for n in self.q_lens:
            self.q_starts.append(self.q_starts[-1] + n)
        self.n_tokens = self.q_starts[-1]
        self.page_size = page_size
        self.compute_dtype = dtype
        self.pad = None


def check_plan(planner, host, plan):
    window = planner.window
    items, merges = plan["items"], plan["merges"]
    assert len(items) == plan["n_small"] + plan["n_large"] + plan["n_long"] and len(merges) == plan["n_merges"]
    seen = {}       # row -> list of (key range seen, partial slot)
    for it in items:
        s, row0, nq = int(it[SEQ]), int(it[ROW]), int(it[NQ])
        assert nq > 0 and host.q_starts[s] <= row0 and row0 + nq <= host.q_starts[s + 1]
        assert int(it[POS]) == host.past_lens[s] + (row0 - host.q_starts[s])
        for t in range(nq):
            pos = int(it[POS]) + t
            lo = max(int(it[KB]), pos - window + 1 if window else 0)
            hi = min(int(it[KE]), pos + 1)
            slot = int(it[PARTIAL]) + t if it[PARTIAL] >= 0 else -1
            seen.setdefault(row0 + t, []).append((lo, hi, slot))
    assert sorted(seen) == list(range(host.n_tokens))
    merged = {int(m[0]): m for m in merges}
    slots_used = set()
    for s in range(host.n_seqs):
        for row in range(host.q_starts[s], host.q_starts[s + 1]):
            pos = host.past_lens[s] + row - host.q_starts[s]
            first = max(0, pos - window + 1) if window else 0
            runs = sorted((lo, hi, slot) for lo, hi, slot in seen[row] if hi > lo)
            # the runs tile [first, pos] exactly
            assert runs[0][0] == first and runs[-1][1] == pos + 1, (row, runs)
            assert all(a[1] == b[0] for a, b in zip(runs, runs[1:])), (row, runs)
            if len(seen[row]) == 1:
                assert seen[row][0][2] == -1 and row not in merged
            else:
                m = merged[row]
                assert int(m[2]) == len(seen[row])
                want = [int(m[1]) + i * int(m[3]) for i in range(int(m[2]))]
                # the merge names the slots in the order of the keys
                assert [slot for _, _, slot in sorted(seen[row])] == want
                assert not slots_used & set(want)
                slots_used |= set(want)
    assert not slots_used or max(slots_used) < plan["n_partial"]
    if plan["mfma"]:
        large = items[plan["n_small"]:]
        covered = []
        for first, count in plan["groups"]:
            assert 1 <= count <= 4
            tiles = large[first:first + count]
            assert len({int(t[SEQ]) for t in tiles}) == 1
            assert all(int(a[POS]) + int(a[NQ]) == int(b[POS]) for a, b in zip(tiles, tiles[1:]))
            covered += list(range(first, first + count))
        assert sorted(covered) == list(range(len(large)))  # every tile in exactly one group
        spans = [int(large[f + n - 1][KE]) - int(large[f][KB]) for f, n in plan["groups"]]
        assert spans == sorted(spans)  # ascending by keys: the kernel starts from the back, longest first
    else:
        assert plan["n_groups"] == 0


@pytest.mark.parametrize("dtype, page_size", [(torch.bfloat16, 16), (torch.float32, 16), (torch.bfloat16, 3)])
@pytest.mark.parametrize("heads, kv, hd, window", [(28, 4, 128, None), (4, 4, 64, None), (6, 2, 32, 100), (20, 1, 256, 700),
                                                   (16, 8, 48, None)])
def test_plans_cover_every_key_once(dtype, page_size, heads, kv, hd, window):
    rng = random.Random(heads * 131 + hd + (window or 0))
    planner = AttentionPlanner(heads, kv, hd, window)
    planner.compute_units = rng.choice([0, 0, 64, 256])
    assert planner.uses_mfma(dtype, page_size) == (dtype == torch.bfloat16 and page_size % 4 == 0 and hd % 16 == 0)
    for _ in range(25):
        seqs = [(rng.choice([0, 0, 1, 15, 16, 255, 600, 1023, 1024, 2500, 5000]),
                 rng.choice([1, 1, 1, 2, 3, 5, 16, 17, 64, 130, 700])) for _ in range(rng.randint(1, 6))]
        host = Host(seqs, page_size, dtype)
        plan = planner.plan(host)
        check_plan(planner, host, plan)
        # with no compute units to fill, a request is cut the same way alone as in the batch;
        # portions longer than a small item always are
        small_tokens = planner.geometry(plan["mfma"])[0]
        for s, (p, n) in enumerate(seqs):
            if planner.compute_units and n <= small_tokens:
                continue
            alone = planner.plan(Host([(p, n)], page_size, dtype))
            mine = [it for it in plan["items"] if it[SEQ] == s]
            theirs = list(alone["items"])
            assert len(mine) == len(theirs)
            key = lambda it: (int(it[ROW]), int(it[KB]))
            for a, b in zip(sorted(mine, key=key), sorted(theirs, key=key)):
                assert int(a[ROW]) - host.q_starts[s] == int(b[ROW])
                assert [int(a[i]) for i in (NQ, POS, KB, KE)] == [int(b[i]) for i in (NQ, POS, KB, KE)]
                assert (a[PARTIAL] >= 0) == (b[PARTIAL] >= 0)


def test_decode_items_shorten_while_compute_units_are_idle():
    planner = AttentionPlanner(28, 4, 128, None)
    planner.compute_units = 256
    # (items halve while the halves' workgroups number at most the units, and between that length and its half
    # they take the shortest multiple of 32 keys that still does: 12 requests of 1,500 keys in 5 items of 320)
    for n_requests, keys, split, waves in ((8, 640, 128, 1), (1, 3550, 128, 1), (64, 640, 1024, 8), (8, 16000, 1024, 8),
                                           (20, 3000, 1024, 8), (12, 1500, 320, 4), (48, 600, 1024, 8), (8, 3550, 448, 4),
                                           (32, 600, 1024, 8), (24, 600, 1024, 8), (16, 640, 160, 2)):
        host = Host([(keys - 1, 1)] * n_requests, 16, torch.bfloat16)
        assert planner.split_keys(host, True) == split
        plan = planner.plan(host)
        check_plan(planner, host, plan)
        assert plan["n_small"] == n_requests * -(-keys // split)
        assert plan["waves"] == waves  # one wave per 128 keys of the longest item, a power of two
        assert plan["n_merges"] == (n_requests if keys > split else 0)
    # requests that by themselves give every unit a workgroup stay whole, however long: no item of 16 keys and no
    # merge for requests that have just passed 1,024; fewer long requests take the longest items of which the
    # full ones still number the units
    # (where the workgroups of such items would leave the last of their rounds over the units mostly empty, or
    # long items leave the units half empty, the items shorten: 16 requests of 9,000 keys in 8 items of 1,152 and
    # not in 4 of 2,048 and one of 808; one request of 100,000 keys in 125 items of 800, not 98 of 1,024; the four
    # keys by which 48 requests have passed 4,096 do not count as workgroups, and whole requests stay whole)
    for n_requests, keys, split, items in ((64, 1040, 2048, 1), (64, 3500, 4096, 1), (80, 2000, 2048, 1), (64, 16000, 16384, 1),
                                           (48, 2000, 1024, 2), (48, 4100, 2048, 3), (32, 3500, 1024, 4), (16, 9000, 1152, 8),
                                           (8, 33000, 2112, 16), (1, 100000, 800, 125)):
        host = Host([(keys - 1, 1)] * n_requests, 16, torch.bfloat16)
        assert planner.split_keys(host, True) == split
        plan = planner.plan(host)
        check_plan(planner, host, plan)
        assert plan["n_small"] == n_requests * items and plan["waves"] == 8
        assert plan["n_merges"] == (n_requests if items > 1 else 0)
        bucket = planner.graph_bucket(host)
        assert bucket[0] >= plan["n_small"] and bucket[1] == 8
    # one very long request among short ones is cut, the short ones stay whole
    host = Host([(599, 1)] * 63 + [(99999, 1)], 16, torch.bfloat16)
    assert planner.split_keys(host, True) == 2048
    plan = planner.plan(host)
    check_plan(planner, host, plan)
    assert plan["n_small"] == 63 + 49 and plan["n_merges"] == 1
    planner.fill_rounds = False  # (without the shortening: the longest items that the rule above allows)
    assert planner.split_keys(host, True) == 4096
    planner.fill_rounds = True
    wide = AttentionPlanner(40, 8, 128, None)
    wide.compute_units = 256
    for n_requests, keys, split in ((8, 16000, 2048), (8, 16500, 2112), (32, 2300, 4096), (16, 4000, 1024), (8, 640, 160)):
        assert wide.split_keys(Host([(keys - 1, 1)] * n_requests, 16, torch.bfloat16), True) == split
    planner.long_items = False
    assert planner.split_keys(Host([(3499, 1)] * 64, 16, torch.bfloat16), True) == 1024
    planner.long_items = True
    # the float32-arithmetic kernel: 256 keys an item on a full device, down to 64 (two passes of 32) on an idle one
    for n_requests, keys, split in ((1, 5000, 64), (8, 640, 64), (64, 640, 256), (4, 2000, 128), (16, 2000, 256)):
        host = Host([(keys - 1, 1)] * n_requests, 16, torch.float32)
        assert planner.split_keys(host, False) == split
        plan = planner.plan(host)
        check_plan(planner, host, plan)
        assert plan["n_small"] == n_requests * -(-keys // split) and plan["waves"] == 1


def test_graph_bucket_pads_plans_of_decode_steps():
    planner = AttentionPlanner(28, 4, 128, None)
    planner.compute_units = 256
    for lens in ([640] * 8, [5, 900, 1500, 3000], [2047, 2048, 2049]):
        host = Host([(p, 1) for p in lens], 16, torch.bfloat16)
        bucket = planner.graph_bucket(host)
        assert bucket is not None and bucket[0] >= len(lens)
        host.pad = {planner.key: bucket}
        plan = planner.plan(host)
        assert plan["n_small"] == bucket[0] and plan["n_large"] == 0 and plan["waves"] == bucket[1]
        # (the length of the items is no part of what the graph fixes: a batch keeps its graph while its requests grow)
        assert sum(1 for it in plan["items"] if it[NQ] > 0) <= bucket[0]
        real = [it for it in plan["items"] if it[NQ] > 0]
        assert sum(int(it[KE]) - int(it[KB]) for it in real) == sum(p + 1 for p in lens)
        if bucket[0] > len(lens):
            assert plan["n_merges"] == len(lens)  # every row gets a merge entry, empty where none is needed
    # a step with a portion is no decode step
    assert planner.graph_bucket(Host([(10, 1), (0, 40)], 16, torch.bfloat16)) is None


def test_the_short_tile_at_the_end_of_a_long_portion_stays_with_its_group():
    """40 query heads on 8 kv heads give tiles of six tokens: a portion of 2,048 tokens ends with a tile
    of two.  That tile is the last of its group of four, not a small item of its own (which would
    walk thousands of keys in one workgroup a kv head while the device idles)."""
    planner = AttentionPlanner(40, 8, 128, None)
    host = Host([(4096, 2048), (0, 1)], 16, torch.bfloat16)
    plan = planner.plan(host)
    check_plan(planner, host, plan)
    small, large, most = planner.geometry(True)
    assert large == 6 and 2048 % large == 2
    items, groups = plan["items"], plan["groups"]
    assert plan["n_small"] == 1 and int(items[0][SEQ]) == 1          # the decoded token of the other request
    tiles = items[plan["n_small"]:]
    assert len(tiles) == -(-2048 // large) and int(tiles[-1][NQ]) == 2
    covered = sorted(i for g in groups for i in range(int(g[0]), int(g[0]) + int(g[1])))
    assert covered == list(range(len(tiles))), "every tile, the short one too, is in a group"
    last = max(groups, key=lambda g: int(g[0]) + int(g[1]))
    assert int(last[0]) + int(last[1]) == len(tiles) and int(last[1]) >= 2
