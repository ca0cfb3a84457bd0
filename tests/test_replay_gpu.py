"""Replay through bin/trace_run: the same requests whole, with the last 32 tokens decoded one by
one, in portions of changing size, and mixed with other requests in a pool so small that pages
are used again; in float32 and bfloat16; all against the plain implementation."""

import json
import random

import numpy as np
import pytest
import torch

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 11, 17, 64, 100, 128, 33], "B": [1, 7, 33, 64, 90, 250, 129]}
PORTIONS = [7, 2, 16, 3, 2, 33, 5, 2, 64, 9]


def requests_of(name):
    vocab = helpers.TINY[name][0]["vocab_size"]
    return {f"{name.lower()}{i}": helpers.token_ids(vocab, n, seed=i + 10 * (name == "B"))
            for i, n in enumerate(LENGTHS[name])}


def build_families(reqs):
    """One trace holding the four families one after the other.  Request ids get a suffix per
    family; returns the builder and {family: {trace id: request name}}."""
    tb = helpers.TraceBuilder()
    fam = {"whole": {}, "decode": {}, "portions": {}, "mixed": {}}
    peak = 0
    for name, ids in reqs.items():  # 1. whole and alone
        rid = name + ".w"
        fam["whole"][rid] = name
        tb.step([(rid, ids, range(len(ids)))], end=[rid])
        peak = max(peak, helpers.round64(len(ids)))
    for name, ids in reqs.items():  # 2. most of it in one step, the last 32 one by one
        rid = name + ".d"
        fam["decode"][rid] = name
        head = max(len(ids) - 32, 1)
        tb.step([(rid, ids[:head], [head - 1])])
        for t in range(head, len(ids)):
            tb.step([(rid, ids[t:t + 1], [0])], end=[rid] if t == len(ids) - 1 else [])
        if head == len(ids):
            tb.step([], end=[rid])
    for k, (name, ids) in enumerate(reqs.items()):  # 3. portions of changing size, down to two
        rid = name + ".p"
        fam["portions"][rid] = name
        i, j = 0, k
        while i < len(ids):
            n = min(PORTIONS[j % len(PORTIONS)], len(ids) - i)
            want = range(n) if (j % 3 or i + n == len(ids)) else []  # some portions ask for nothing
            tb.step([(rid, ids[i:i + n], want)], end=[rid] if i + n == len(ids) else [])
            i += n
            j += 1
    # 4. mixed: up to four live requests, portions of some beside single tokens of others
    rng = random.Random(7)
    pending = [(name + sfx, name) for sfx in (".m", ".n", ".o") for name in reqs]
    live, fed = {}, {}
    while pending or live:
        while pending and len(live) < 4:
            rid, name = pending.pop(0)
            live[rid] = reqs[name]
            fed[rid] = 0
            fam["mixed"][rid] = name
        entries, end = [], []
        for rid, ids in list(live.items()):
            if rng.random() < 0.15 and len(live) > 1:
                continue  # left out of this step, goes on later
            left = len(ids) - fed[rid]
            decode_from = max(len(ids) - 24, len(ids) // 2)
            n = 1 if fed[rid] >= decode_from else min(left, rng.choice([2, 3, 5, 8, 16, 31]), decode_from - fed[rid])
            n = max(n, 1)
            entries.append((rid, ids[fed[rid]:fed[rid] + n], range(n)))
            fed[rid] += n
            if fed[rid] == len(ids):
                end.append(rid)
        if not entries:
            continue
        peak = max(peak, sum(helpers.round64(fed[r]) for r in live))
        tb.step(entries, end=end)
        for rid in end:
            del live[rid]
    return tb, fam, peak


@pytest.fixture(scope="module")
def replays(model_dirs, tmp_path_factory):
    out = {}
    for name in ("A", "B"):
        reqs = requests_of(name)
        tb, fam, peak = build_families(reqs)
        cfg, w = plain.read_config(model_dirs[name]), plain.read_weights(model_dirs[name])
        ref = {r: plain.forward(cfg, w, ids).numpy() for r, ids in reqs.items()}
        for dtype in ("float32", "bfloat16"):
            print(f"replay {name} {dtype}: {len(tb.steps)} steps, pool for {peak} tokens", flush=True)
            out_dir = tmp_path_factory.mktemp(f"out_{name}_{dtype}")
            res = helpers.run_trace(model_dirs[name], dtype, tb.steps, peak, out_dir)
            stats = json.loads((out_dir / "cache_stats.json").read_text())
            out[(name, dtype)] = (helpers.collect(tb, res), fam, ref, reqs, stats)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("family", ["whole", "decode", "portions", "mixed"])
def test_family_matches_plain(replays, name, dtype, family):
    per, fam, ref, reqs, _ = replays[(name, dtype)]
    assert fam[family]
    checked = clear = 0
    for rid, req in fam[family].items():
        rows = per.get(rid, {})
        if family in ("whole", "mixed"):
            assert sorted(rows) == list(range(len(reqs[req]))), f"{rid}: every position was asked for"
        if family == "decode":
            assert len(rows) == min(33, len(reqs[req]))
        pos = sorted(rows)
        got = np.stack([rows[p] for p in pos])
        clear += helpers.assert_close_to_plain(got, ref[req][pos], dtype, f"{name} {dtype} {family} {rid}")[0]
        checked += len(pos)
    assert checked > 100
    if dtype == "float32":
        print(f"{name} {family}: argmax compared on {clear} of {checked} rows")
        assert 2 * clear >= checked, f"the argmax was compared on {clear} of {checked} rows only"


@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_families_agree_beyond_rounding_only(replays, name):
    """How the tokens were cut, what else was in the batch and which pages were used changes
    the float32 logits by rounding only."""
    per, fam, ref, reqs, _ = replays[(name, "float32")]
    whole = {req: per[rid] for rid, req in fam["whole"].items()}
    for family in ("decode", "portions", "mixed"):
        for rid, req in fam[family].items():
            for pos, row in per[rid].items():
                assert np.abs(row - whole[req][pos]).max() <= 2e-5, f"{family} {rid} position {pos}"


def test_pages_were_used_again(replays):
    """From the allocator's own counters, written by the replay when its input ends: more pages
    were handed out than the pool has, most pages more than once, and all came back."""
    for (name, dtype), (_, _, _, _, stats) in replays.items():
        for g in stats["groups"]:
            assert g["pages_issued"] > 2 * g["pages"], (name, dtype, g)
            assert g["pages_issued_again"] > g["pages"] // 2, (name, dtype, g)
            assert g["free_at_end"] == g["pages"], (name, dtype, g)


def test_refusals_and_empty_steps(model_dirs, tmp_path):
    """A step with no entries, a request left out of steps, and ending a request twice over."""
    ids = helpers.token_ids(256, 20, 99)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": ids[:10], "want": []}], "end": []},
             {"step": 1, "entries": [], "end": []},
             {"step": 2, "entries": [{"id": "y", "tokens": ids[:3], "want": [2]}], "end": ["y"]},
             {"step": 3, "entries": [{"id": "x", "tokens": ids[10:], "want": [9]}], "end": ["x"]}]
    res = helpers.run_trace(model_dirs["A"], "float32", steps, 128, tmp_path / "o")
    ref = plain.forward_dir(model_dirs["A"], ids).numpy()
    assert sorted(res) == [2, 3]
    helpers.assert_close_to_plain(res[3], ref[19:20], "float32", "left out and resumed")
    helpers.assert_close_to_plain(res[2], ref[2:3], "float32", "other request")
