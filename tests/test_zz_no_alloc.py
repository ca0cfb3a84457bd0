"""The entry point that allocates nothing (split-key attention and its merge with the partial
records in the library's own buffer), called through ctypes, against the existing entry points
(attention with a caller's workspace, then the merge) on two calls in a row, the second with a
smaller input.

"Allocates nothing" is observed in three ways, none of which sees everything: torch's caching
allocator counts no new block (that sees torch's own allocations only); the device's free memory
as the driver reports it (``torch.cuda.mem_get_info``, which a ``hipMalloc`` inside the library
would move) is the same before and after every call but the process's first, which may pay for
loading the library's code and for ``hipGetSymbolAddress``; and one call is made while its stream
is being captured into a graph, where an allocation is an error, and the graph's replay gives the
same bits.  What is not observed: host memory."""

import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _existing(ops, case, heads, kv, hd, mfma):
    q = case["q"].cuda()
    plan = case["plan"]
    t = q.shape[0]
    out = torch.zeros((t, heads * hd), dtype=q.dtype).cuda()
    partials = torch.empty(max(plan["n_partial"], 1) * heads * (hd + 2), dtype=torch.float32).cuda()
    items = torch.from_numpy(plan["items"]).cuda()
    pools = (case["k_pool"].cuda(), case["v_pool"].cuda(), case["tables"].cuda())
    args = (items, plan["n_small"], out, partials, heads, kv, hd, None, 1.0 / math.sqrt(hd), t)
    if mfma:
        ops.attention_mfma(q, heads * hd, *pools, *args, large=False, waves=plan["waves"])
    else:
        ops.attention_scalar(q, heads * hd, *pools, *args)
    ops.attention_merge(partials, torch.from_numpy(plan["merges"]).cuda(), plan["n_merges"], out, heads, hd)
    return out


_calls = {"n": 0}


def _static(ops, case, heads, kv, hd, mfma, n_partial_slots=None, capture=False):
    lib = ops.load()
    q = case["q"].cuda()
    plan = case["plan"]
    t = q.shape[0]
    out = torch.zeros((t, heads * hd), dtype=q.dtype).cuda()
    items = torch.from_numpy(plan["items"]).cuda()
    merges = torch.from_numpy(plan["merges"]).cuda()
    k_pool, v_pool, tables = case["k_pool"].cuda(), case["v_pool"].cuda(), case["tables"].cuda()
    call = lambda: lib.fsie_attention_split_static(
        q.data_ptr(), heads * hd, k_pool.data_ptr(), v_pool.data_ptr(), tables.data_ptr(), tables.shape[1],
        items.data_ptr(), plan["n_small"], merges.data_ptr(), plan["n_merges"],
        plan["n_partial"] if n_partial_slots is None else n_partial_slots, out.data_ptr(), heads, kv, hd,
        k_pool.shape[2], 0, ctypes.c_float(1.0 / math.sqrt(hd)), 1 if q.dtype == torch.bfloat16 else 0, int(mfma),
        plan["waves"], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    if capture:
        # while the stream is captured an allocation (or anything else that waits for the device) is an
        # error that the call would report; the kernels run when the graph is replayed
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            rc = call()
        assert float(out.float().abs().max()) == 0.0, "a captured call runs nothing"
        graph.replay()
        torch.cuda.synchronize()
        return rc, out
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]
    rc = call()
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    if _calls["n"] > 0:  # (the process's first call may load the library's code onto the device)
        assert torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed over the call"
    _calls["n"] += 1
    return rc, out


@pytest.mark.parametrize("dtype, mfma", [(torch.bfloat16, True), (torch.float32, False)])
def test_split_attention_in_the_librarys_own_buffer(dtype, mfma):
    from from_scratch_inference_engine_amd import ops
    from test_kernels_gpu import paged_case

    heads, kv, hd, page = 28, 4, 128, 16
    first = [(2500, 1), (600, 1), (40, 1), (1300, 2)]
    second = [(700, 1)]
    for seqs, seed in ((first, 1), (second, 2)):
        case = paged_case(seqs, heads, kv, hd, page, dtype, seed=seed, scalar=not mfma)
        plan = case["plan"]
        assert plan["mfma"] == mfma and plan["n_merges"] > 0 and plan["n_large"] == 0
        want = _existing(ops, case, heads, kv, hd, mfma)
        rc, got = _static(ops, case, heads, kv, hd, mfma)
        assert rc == 0, ops.load().fsie_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"{seqs}: the two entry points give other bits"
        assert got.float().abs().max() > 0
        rc, got = _static(ops, case, heads, kv, hd, mfma, capture=True)
        assert rc == 0, ops.load().fsie_last_error()
        assert torch.equal(got, want), f"{seqs}: the call captured into a graph and replayed gives other bits"
    # a table that names slots beyond what the caller said (the first case, one slot short): those
    # records do nothing.  A row whose merge is dropped stays as it was, a row that lost an item
    # but not its merge is not looked at, every other row is as before.
    case = paged_case(first, heads, kv, hd, page, dtype, seed=1, scalar=not mfma)
    plan, limit = case["plan"], case["plan"]["n_partial"] - 1
    want = _existing(ops, case, heads, kv, hd, mfma)
    rc, got = _static(ops, case, heads, kv, hd, mfma, n_partial_slots=limit)
    assert rc == 0, ops.load().fsie_last_error()
    lost = [(int(it[6]), int(it[6] + it[2])) for it in plan["items"][:plan["n_small"]] if it[6] >= 0 and it[6] + it[2] > limit]
    slots_of = lambda m: range(int(m[1]), int(m[1] + (m[2] - 1) * m[3]) + 1, max(int(m[3]), 1))
    dropped = sorted(int(m[0]) for m in plan["merges"] if max(slots_of(m)) >= limit)
    touched = {int(m[0]) for m in plan["merges"] if any(a <= s < b for s in slots_of(m) for a, b in lost)}
    kept = [r for r in range(got.shape[0]) if r not in touched and r not in dropped]
    assert lost and dropped and len(kept) >= 3
    assert float(got[dropped].float().abs().max()) == 0.0
    assert torch.equal(got[kept], want[kept])
    # more partial records than the buffer holds: refused, nothing runs
    slots = ops.load().fsie_static_scratch_bytes() // (heads * (hd + 2) * 4) + 1
    rc, _ = _static(ops, case, heads, kv, hd, mfma, n_partial_slots=slots)
    assert rc != 0 and b"the library's buffer" in ops.load().fsie_last_error()
