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


# ------------------------------------------------------------------ running one step ahead
def launch(m, items):
    """Queue a step as the engine does: pages reserved and lengths advanced at once."""
    assert m.can_reserve([(it.seq.cache, len(it.tokens)) for it in items])
    for it in items:
        m.reserve(it.seq.cache, len(it.tokens))
        m.commit(it.seq.cache, len(it.tokens))
    return items


def run_pipelined(m, s, token_of, ahead_log=None):
    """The engine's loop with one step queued ahead; the token of a sample depends only on the
    request and on how many it has, as in ``run_step``."""
    pending, steps = None, 0
    while s.has_work() or pending is not None:
        if pending is not None and not any(it.wants_logits and it.seq.status == SeqStatus.Running for it in pending):
            pending = None
        if pending is None:
            items = s.schedule()
            if not items:
                break
            pending = launch(m, items)
        items = pending
        # the samples "on the device": fixed before the next step is queued (the step before this
        # one has been read by now, so a sample's index is the length of the output)
        samples = [token_of(it.seq, len(it.seq.output)) if it.wants_logits else None for it in items]
        nxt = s.lookahead(items)
        pending = launch(m, nxt) if nxt is not None else None
        if ahead_log is not None:
            ahead_log.append(nxt is not None)
        s.finish_step(items, samples)
        m.check_invariants()
        steps += 1
        assert steps < 1000
    return steps


def test_lookahead_only_when_the_next_step_is_certain():
    m, s = make(num_pages=32, budget=6)
    a = s.add_request(Request([1, 2, 3, 4, 5, 6, 7, 8], max_tokens=4))
    items = launch(m, s.schedule())
    assert not items[0].wants_logits and s.lookahead(items) is None      # still in its prompt
    s.finish_step(items, [None])
    items = launch(m, s.schedule())
    assert items[0].wants_logits
    b = s.add_request(Request([9], max_tokens=1))
    assert s.lookahead(items) is None                                    # somebody waits to be admitted
    s.finish_step(items, [100])
    items = launch(m, s.schedule())                                      # a decodes, b's prompt
    assert [it.seq.id for it in items] == [a, b]
    assert s.lookahead(items) is None                                    # b's pending sample is its last
    s.finish_step(items, [101, 200])
    assert s.sequences[b].status == SeqStatus.Finished
    items = launch(m, s.schedule())
    assert s.lookahead(items) is not None                                # a alone: third of four


def test_lookahead_steps_and_limits():
    m, s = make(num_pages=32)
    a = s.add_request(Request([1, 2, 3], max_tokens=4))
    b = s.add_request(Request([4], max_tokens=6))
    items = launch(m, s.schedule())
    nxt = s.lookahead(items)
    assert nxt is not None and [(it.seq.id, it.tokens, it.wants_logits, it.ahead) for it in nxt] == \
        [(a, [0], True, True), (b, [0], True, True)]
    launch(m, nxt)
    assert s.sequences[a].remaining == -1                                # one token ahead of its output
    s.finish_step(items, [100, 200])
    assert s.sequences[a].remaining == 0
    nxt2 = s.lookahead(nxt)
    assert nxt2 is not None
    launch(m, nxt2)
    s.finish_step(nxt, [101, 201])
    nxt3 = s.lookahead(nxt2)                                             # a's pending sample is its third of four
    assert nxt3 is not None
    launch(m, nxt3)
    s.finish_step(nxt2, [102, 202])
    assert s.lookahead(nxt3) is None                                     # a's pending sample is its last
    s.finish_step(nxt3, [103, 203])
    assert s.sequences[a].status == SeqStatus.Finished and s.sequences[b].output == [200, 201, 202, 203]
    m.check_invariants()


def test_lookahead_needs_a_page_for_every_request():
    m, s = make(num_pages=3, page_size=2)
    s.add_request(Request([1, 2], max_tokens=3))
    s.add_request(Request([3, 4], max_tokens=3))
    items = launch(m, s.schedule())
    assert len(items) == 2 and m.free_pages() == 1
    assert s.lookahead(items) is None                                    # both need a new page for one more token


def test_pipelined_loop_gives_the_same_outputs_and_frees_everything():
    def token_of(seq, index):
        return 7 if (seq.id * 5 + index) % 11 == 3 else 100 + index     # some requests meet their eos

    outs = []
    for pipelined in (False, True):
        m, s = make(num_pages=24, page_size=2, budget=9, max_batch=4)
        for i in range(10):
            n = 1 + (i * 3) % 6
            s.add_request(Request(list(range(1, n + 1)), max_tokens=1 + (i * 7) % 9, eos_id=7))
        log = []
        if pipelined:
            run_pipelined(m, s, token_of, log)
            assert any(log) and not all(log)
        else:
            while s.has_work():
                run_step(m, s, token_of=lambda seq: token_of(seq, len(seq.output)))
        assert m.free_pages() == 24 and m.free_slots == 4
        outs.append({sid: list(q.output) for sid, q in s.sequences.items()})
        assert all(q.status == SeqStatus.Finished for q in s.sequences.values())
    assert outs[0] == outs[1]
    assert any(o[-1] == 7 and len(o) > 1 for o in outs[0].values())     # an eos was found one step late


def test_no_more_running_requests_than_a_step_has_tokens_for():
    """max_batch above the token budget is cut to it: six requests, three tokens a step; the three
    that run each decode in every step, the others are admitted as those finish."""
    m, s = make(num_pages=64, page_size=2, budget=3, max_batch=6)
    assert s.max_batch == 3
    ids = [s.add_request(Request([1 + i], max_tokens=4)) for i in range(6)]
    seen = []
    while s.has_work():
        items = launch(m, s.schedule())
        assert 0 < sum(len(it.tokens) for it in items) <= 3
        running = [q for q in s.running]
        assert sorted(it.seq.id for it in items) == sorted(running)  # nobody who runs is left out
        seen.append([it.seq.id for it in items])
        s.finish_step(items, [50] * len(items))
    assert seen[0] == ids[:3] and seen[-1] == ids[3:]
    assert all(len(s.sequences[i].output) == 4 for i in ids)
    m.check_invariants()
