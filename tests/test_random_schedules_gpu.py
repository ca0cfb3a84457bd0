"""Random schedules through the step function, against the plain implementation: up to four live
requests, portions of any size beside decoded tokens, logits wanted at random places, a pool so
small that requests are ended to make room and their pages are used again.  After every step the
cache manager's invariants hold."""

import random

import numpy as np
import pytest

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed, page_size, num_pages", [(0, 4, 40), (1, 16, 10), (2, 8, 200)])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_schedule_matches_plain(model_dirs, name, dtype, seed, page_size, num_pages):
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    d = model_dirs[name]
    cfg = plain.read_config(d)
    vocab, longest = cfg["vocab_size"], cfg.get("max_position_embeddings", 1 << 30)
    rng = random.Random(1000 * seed + len(name))
    runner = Runner(load_model(d, dtype=dtype), page_size=page_size, num_pages=num_pages, max_requests=4)
    live, next_id, checked, reused = {}, 0, 0, 0
    for step in range(70):
        while len(live) < 4 and rng.random() < 0.5:
            n = min(rng.choice([1, 2, 3, 7, 16, 17, 33, 64, 100]) + rng.randint(0, 12), longest)
            ids = helpers.token_ids(vocab, n, 5000 + 100 * seed + next_id)
            live[next_id] = {"ids": ids, "fed": 0, "cache": runner.manager.open(next_id), "ref": None}
            next_id += 1
        if not live:
            continue
        chosen = [k for k in live if rng.random() < 0.8] or [next(iter(live))]
        entries, meta = [], []
        for k in chosen:
            r = live[k]
            n = min(len(r["ids"]) - r["fed"], rng.choice([1, 1, 1, 2, 3, 5, 16, 31, 64]))
            want = sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))
            entries.append(StepEntry(r["cache"], r["ids"][r["fed"]:r["fed"] + n], want))
            meta.append((k, r["fed"], want))
        if not runner.manager.can_reserve((e.cache, len(e.tokens)) for e in entries):
            k = max(live, key=lambda k: live[k]["fed"])  # no room: the longest request ends, its pages come back
            runner.manager.close(live.pop(k)["cache"])
            reused += 1
            continue
        out = runner.step(entries).float().cpu().numpy()
        row = 0
        for (k, fed0, want), e in zip(meta, entries):
            r = live[k]
            if want and r["ref"] is None:
                r["ref"] = plain.forward_dir(d, r["ids"]).numpy()
            for w in want:
                helpers.assert_close_to_plain(out[row:row + 1], r["ref"][fed0 + w:fed0 + w + 1], dtype,
                                              f"{name} {dtype} seed {seed} step {step} request {k} position {fed0 + w}")
                row += 1
                checked += 1
            r["fed"] += len(e.tokens)
        for k in [k for k in live if live[k]["fed"] == len(live[k]["ids"])]:
            runner.manager.close(live.pop(k)["cache"])
        runner.manager.check_invariants()
    assert checked > 50
    if num_pages * page_size <= 160:
        assert reused > 0  # the small pools did run out
        alloc = runner.manager.allocators[0]
        assert alloc.pages_issued > num_pages and len(alloc.pages_issued_again()) > num_pages // 2
