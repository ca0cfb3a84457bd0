"""The scheduler's decisions, on the CPU: admission, portions under a token budget, decoding,
finishing and freeing, and what happens when pages run out."""

import pytest

from from_scratch_inference_engine_amd.cache import CacheManager, PagedNeed
from from_scratch_inference_engine_amd.engine.scheduler import Request, Scheduler, SeqStatus
from from_scratch_inference_engine_amd.sampling import SamplingParams


def make(num_pages, page_size=4, max_batch=8, budget=2048, chunk=None, max_position=0):
    m = CacheManager([PagedNeed(2, 16)], page_size=page_size, num_pages=num_pages, max_requests=max_batch)
    return m, Scheduler(m, max_batch=max_batch, max_tokens_per_step=budget, prefill_chunk=chunk, max_position=max_position)


def run_step(m, s, token_of=lambda seq: 100 + len(seq.output)):
    """What the engine does around a schedule: reserve, commit, hand back sampled tokens."""
    items = s.schedule()
    assert m.can_reserve([(it.seq.cache, len(it.tokens)) for it in items])
    for it in items:
        m.reserve(it.seq.cache, len(it.tokens))
        m.commit(it.seq.cache, len(it.tokens))
    s.finish_step(items, [token_of(it.seq) if it.wants_logits else None for it in items])
    m.check_invariants()
    return items


def test_prefill_then_decode_then_finish_and_free():
    m, s = make(num_pages=16)
    a = s.add_request(Request([1, 2, 3, 4, 5], SamplingParams(0.0), max_tokens=3))
    items = run_step(m, s)
    assert [(it.seq.id, it.tokens, it.wants_logits) for it in items] == [(a, [1, 2, 3, 4, 5], True)]
    assert s.sequences[a].output == [100] and s.sequences[a].status == SeqStatus.Running
    items = run_step(m, s)
    assert items[0].tokens == [100] and items[0].wants_logits  # decoding feeds the last output token
    items = run_step(m, s)
    assert s.sequences[a].output == [100, 101, 102] and s.sequences[a].status == SeqStatus.Finished
    assert m.free_pages() == 16 and m.free_slots == 8 and not s.has_work()
    assert s.schedule() == []


def test_eos_is_kept_and_stops():
    # tests/cpp/test_engine.cpp:130-141
    m, s = make(num_pages=16)
    a = s.add_request(Request([1, 2], max_tokens=10, eos_id=7))
    run_step(m, s, token_of=lambda seq: 7)
    assert s.sequences[a].output == [7] and s.sequences[a].status == SeqStatus.Finished and m.free_pages() == 16


def test_token_budget_cuts_prompts_into_portions_and_decodes_first():
    m, s = make(num_pages=64, budget=8)
    a = s.add_request(Request(list(range(1, 4)), max_tokens=4))        # 3 tokens
    b = s.add_request(Request(list(range(10, 30)), max_tokens=2))      # 20 tokens
    items = run_step(m, s)
    assert [(it.seq.id, len(it.tokens), it.wants_logits) for it in items] == [(a, 3, True), (b, 5, False)]
    items = run_step(m, s)  # a decodes (1 token, first), b gets the remaining 7 of the budget
    assert [(it.seq.id, len(it.tokens), it.wants_logits) for it in items] == [(a, 1, True), (b, 7, False)]
    assert items[1].tokens == list(range(15, 22))
    items = run_step(m, s)
    assert [(it.seq.id, len(it.tokens)) for it in items] == [(a, 1), (b, 7)]
    items = run_step(m, s)  # a's 4th and last token; b's last prompt token wants logits
    assert [(it.seq.id, len(it.tokens), it.wants_logits) for it in items] == [(a, 1, True), (b, 1, True)]
    assert s.sequences[a].status == SeqStatus.Finished and s.sequences[b].output == [100]
    # prefill_chunk caps a portion below the budget
    m, s = make(num_pages=64, budget=100, chunk=6)
    s.add_request(Request(list(range(20)), max_tokens=1))
    assert [len(run_step(m, s)[0].tokens) for _ in range(4)] == [6, 6, 6, 2]


def test_fcfs_head_of_line_blocks_and_second_request_waits():
    # tests/cpp/test_engine.cpp:75-99: a pool of one page of 8: the second request waits
    m, s = make(num_pages=1, page_size=8)
    a = s.add_request(Request([1, 2, 3], max_tokens=3))
    b = s.add_request(Request([4, 5], max_tokens=2))
    c = s.add_request(Request([6], max_tokens=1))
    items = run_step(m, s)
    assert [it.seq.id for it in items] == [a]
    assert s.sequences[b].status == SeqStatus.Waiting and s.sequences[c].status == SeqStatus.Waiting
    run_step(m, s)
    run_step(m, s)
    assert s.sequences[a].status == SeqStatus.Finished
    items = run_step(m, s)  # b is admitted once a's page is back; c does not overtake b
    assert [it.seq.id for it in items] == [b]
    while s.has_work():
        run_step(m, s)
    assert s.sequences[c].output == [100] and s.preemptions == 0


def test_pages_run_out_preempts_youngest_and_recomputes():
    # tests/cpp/test_engine.cpp:103-128: two pages of 4, two prompts of 4 tokens
    m, s = make(num_pages=2, page_size=4)
    a = s.add_request(Request([1, 2, 3, 4], max_tokens=3))
    b = s.add_request(Request([5, 6, 7, 8], max_tokens=3))
    items = run_step(m, s)
    assert [it.seq.id for it in items] == [a, b] and m.free_pages() == 0
    # both need a new page for their next token, none is free: the youngest (b) goes back
    items = run_step(m, s)
    assert s.preemptions == 1 and [it.seq.id for it in items] == [a]
    assert s.sequences[b].status == SeqStatus.Waiting and s.sequences[b].cache is None
    assert s.sequences[b].output == [100] and list(s.waiting) == [b]
    while s.sequences[a].status != SeqStatus.Finished:
        run_step(m, s)
    items = run_step(m, s)  # b recomputes prompt + its one output token, then goes on
    assert [(it.seq.id, it.tokens, it.wants_logits) for it in items] == [(b, [5, 6, 7, 8, 100], True)]
    while s.has_work():
        run_step(m, s)
    assert s.sequences[b].output == [100, 101, 102] and m.free_pages() == 2


def test_starved_request_is_skipped_while_others_run():
    m, s = make(num_pages=3, page_size=4)
    a = s.add_request(Request([1, 2, 3, 4], max_tokens=4))   # full page: needs a new one to decode
    b = s.add_request(Request([5, 6], max_tokens=2))          # room left in its page
    run_step(m, s)
    hog = m.open("someone else")
    m.reserve(hog, 4)  # takes the last free page
    items = run_step(m, s)
    assert [it.seq.id for it in items] == [b] and s.preemptions == 0  # a is left out, nothing preempted
    assert s.sequences[b].status == SeqStatus.Finished
    m.close(hog)
    items = run_step(m, s)
    assert [it.seq.id for it in items] == [a]


def test_portion_shrinks_to_the_free_pages():
    m, s = make(num_pages=4, page_size=4, budget=64)
    a = s.add_request(Request(list(range(14)), max_tokens=1))
    s._admit()
    hog = m.open("someone else")
    m.reserve(hog, 8)  # 2 pages left: only 8 of the 14 tokens fit now
    items = run_step(m, s)
    assert [(it.seq.id, len(it.tokens), it.wants_logits) for it in items] == [(a, 8, False)]
    assert run_step(m, s) == []  # nothing fits, one request running: no progress, no preemption
    m.close(hog)
    items = run_step(m, s)
    assert [(it.seq.id, len(it.tokens), it.wants_logits) for it in items] == [(a, 6, True)]


def test_refused_at_add():
    m, s = make(num_pages=4, page_size=4, max_position=32)
    with pytest.raises(ValueError, match="empty prompt"):
        s.add_request(Request([]))
    with pytest.raises(ValueError, match="never run"):
        s.add_request(Request(list(range(10)), max_tokens=8))   # 17 tokens > 16 slots
    s.add_request(Request(list(range(10)), max_tokens=7))       # 16 tokens: fits exactly
    m2, s2 = make(num_pages=64, page_size=4, max_position=32)
    with pytest.raises(ValueError, match="max_position_embeddings"):
        s2.add_request(Request(list(range(30)), max_tokens=4))
    with pytest.raises(ValueError, match="max_tokens"):
        s2.add_request(Request([1], max_tokens=0))


def test_max_batch_limits_running():
    m, s = make(num_pages=64, max_batch=2)
    ids = [s.add_request(Request([i + 1], max_tokens=2)) for i in range(4)]
    items = run_step(m, s)
    assert [it.seq.id for it in items] == ids[:2] and len(s.waiting) == 2
    run_step(m, s)
    items = run_step(m, s)
    assert [it.seq.id for it in items] == ids[2:]


def test_many_requests_small_pool_all_finish():
    m, s = make(num_pages=6, page_size=2, budget=7, max_batch=4)
    want = {}
    for i in range(9):
        n = 1 + (i * 3) % 5
        sid = s.add_request(Request(list(range(1, n + 1)), max_tokens=1 + i % 4))
        want[sid] = 1 + i % 4
    steps = 0
    while s.has_work():
        before = (steps, s.preemptions)
        items = run_step(m, s)
        steps += 1
        assert items or s.preemptions > before[1], "a step must make progress"
        assert sum(len(it.tokens) for it in items) <= 7
        assert steps < 500
    for sid, n in want.items():
        assert s.sequences[sid].output == [100 + k for k in range(n)]
    assert m.free_pages() == 6 and m.free_slots == 4
