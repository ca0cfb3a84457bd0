"""The engine against the plain implementation at the layer sizes of Qwen2.5-7B: hidden 3584,
28 query and 4 key/value heads of 128, intermediate 18944, vocabulary 152,064, untied head, page
size 16.  Four layers instead of 28 (named here, so that the test fits the suite's time and the
host's memory: 2.0 billion parameters, 8 GB as float32 for the plain side); every width, and so
every kernel shape of the full model, is the real one.

float32: prompts of 330, 301 and 77 tokens, whole; all but the last 32 tokens in one step and
those one by one; in portions of changing size; and mixed in one pool so small that the second
wave of requests gets the pages of the first.  Within 1e-4 of the plain logits, identical argmax
wherever the plain choice is clear (the reference's own whole-model checks on its device path:
tests/cpp/test_cuda_model.cpp:18-70, 113-218).

bfloat16: the same families.  Random weights give small logits and rounding the activations to
bfloat16 moves them by a few per cent of the largest one, in the plain model as well; so the
bound is stated against that: the engine may differ from the plain float32 logits by at most
twice (largest) and one and a half times (root mean square) what the plain model itself moves
when its activations are rounded to bfloat16 where the engine rounds them, and it picks the
plain token wherever that one leads by more than twice the largest difference.  Decode batches
of 32, 64, 80, 100, 128 and 140 through replayed graphs (rows of 32, 64, 80, 112, 128 and 160: the engine's
own products up to 128 rows, beyond that the library's, its kernels chosen by timing) are checked against
the plain logits in the same way.  One step of 2,048 tokens with the library's kernels chosen by
timing (what the prefill measurement runs) is held to the same bound at 24 of its rows, and
``Engine.generate_batch`` (scheduler, one step ahead, graphs, sampling on the device) must give the
plain greedy tokens in float32 up to the first place where the plain choice is not clear.

The same at the layer sizes of Qwen2.5-14B and -32B (hidden 5120, 40 query and 8 key/value heads of
128, so five heads a group, intermediate 13824, eps 1e-5; two layers, named here): the families
that decode and mix, in both precisions.
"""

import json

import numpy as np
import pytest
import torch

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

LAYERS = 4  # of the 28 that the 7B shape has
WIDE = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 3584,
    "num_hidden_layers": LAYERS, "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "use_sliding_window": False,
}
LAYERS_14B = 2  # of the 48 that the 14B shape has
WIDE_14B = dict(WIDE, hidden_size=5120, num_hidden_layers=LAYERS_14B, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=13824, rms_norm_eps=1e-5, max_position_embeddings=8192)
LENGTHS = [330, 301, 77]
PORTIONS = [7, 2, 16, 3, 2, 33, 5, 2, 64, 9, 130]


def _rounded_plain(cfg, w, ids, rows=None, many_rows=False):
    """The plain model with its activations rounded to bfloat16 where the bfloat16 engine rounds
    them: the inputs of every product, q and k after the rotation, the gated activation.
    ``many_rows``: also what a step of many rows rounds (its products come from the library as
    bfloat16, where steps of up to 128 rows keep float32 partial sums): the result of every product
    but the head's, and the values as the cache keeps them."""
    r16 = lambda t: t.to(torch.bfloat16).float()
    lin, rope, silu, att = plain.linear, plain.rope, plain.silu_mul, plain.attention

    def linear(x, wt, b=None):
        y = lin(r16(x), wt)
        if many_rows and wt.shape[0] != cfg["vocab_size"]:
            y = r16(y)
        return y if b is None else y + b

    plain.linear = linear
    plain.rope = lambda *a, **k: r16(rope(*a, **k))
    plain.silu_mul = lambda g, u: r16(silu(r16(g), r16(u)))
    if many_rows:
        plain.attention = lambda q, k, v, *a, **kw: att(q, k, r16(v), *a, **kw)
    try:
        return plain.forward(cfg, w, ids, rows=rows)
    finally:
        plain.linear, plain.rope, plain.silu_mul, plain.attention = lin, rope, silu, att


def _write_model(folder, raw, seed):
    """bfloat16 values, drawn on the device by the test's own generator, so that both precisions
    and the plain side read the same numbers."""
    from safetensors.torch import save_file

    (folder / "config.json").write_text(json.dumps(raw))
    g = torch.Generator(device="cuda").manual_seed(seed)
    tensors = {}
    for name, shape in sorted(helpers.expected_tensor_shapes(raw).items()):
        t = torch.randn(shape, generator=g, device="cuda") * 0.02
        if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
            t = t + 1.0
        tensors[name] = t.to(torch.bfloat16).cpu()
    save_file(tensors, str(folder / "model.safetensors"))


def _plain_side(d, raw):
    cfg, w = plain.read_config(d), plain.read_weights(d)
    prompts = [helpers.token_ids(raw["vocab_size"], n, 4000 + n) for n in LENGTHS]
    ref = [plain.forward(cfg, w, p) for p in prompts]
    print("plain logits done", flush=True)
    moved = [(_rounded_plain(cfg, w, p) - r) for p, r in zip(prompts, ref)]
    noise = [(m.abs().max().item(), m.pow(2).mean().sqrt().item()) for m in moved]
    print("rounded plain logits done", flush=True)
    return cfg, w, {"dir": d, "prompts": prompts, "ref": ref, "noise": noise}


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    """The model folder at 7B widths and the plain logits."""
    d = tmp_path_factory.mktemp("wide7b")
    _write_model(d, WIDE, 11)
    print("wide model written", flush=True)
    cfg, w, out = _plain_side(d, WIDE)
    # short prompts of the decode batches (graphs): the first eight are compared with the plain model
    out["short"] = [helpers.token_ids(WIDE["vocab_size"], 20 + i % 7 + 12, 5000 + i) for i in range(140)]
    out["short_ref"] = [plain.forward(cfg, w, p) for p in out["short"][:8]]
    # one prompt of 2,048 tokens, its plain logits at 24 places and what rounding alone moves there
    long_ids = helpers.token_ids(WIDE["vocab_size"], 2048, 6000)
    rows = sorted({0, 1, 15, 16, 17, 255, 256, 1023, 1024, 2046, 2047} | set(range(100, 2048, 150)))
    long_ref = plain.forward(cfg, w, long_ids, rows=rows)
    moved = _rounded_plain(cfg, w, long_ids, rows=rows, many_rows=True) - long_ref
    out["long"] = {"ids": long_ids, "rows": rows, "ref": long_ref,
                   "noise": (moved.abs().max().item(), moved.pow(2).mean().sqrt().item())}
    print("plain logits of the 2,048-token prompt done", flush=True)
    # greedy continuations of three short prompts, with the lead of every chosen token
    greedy = []
    for p in out["short"][:3]:
        ids, toks, leads = list(p), [], []
        for _ in range(12):
            last = plain.forward(cfg, w, ids, rows=[len(ids) - 1])[0]
            top2 = last.topk(2)
            toks.append(int(top2.indices[0]))
            leads.append(float(top2.values[0] - top2.values[1]))
            ids.append(toks[-1])
        greedy.append((toks, leads))
    out["greedy"] = greedy
    print("plain greedy continuations done", flush=True)
    del w
    return out


@pytest.fixture(scope="module")
def wide_14b(tmp_path_factory):
    d = tmp_path_factory.mktemp("wide14b")
    _write_model(d, WIDE_14B, 12)
    print("14B-geometry model written", flush=True)
    _, w, out = _plain_side(d, WIDE_14B)
    del w
    return out


def _plans():
    """{family: list of steps; a step is a list of (request key, prompt index, n tokens)}."""
    n = LENGTHS
    whole = [[(f"w{i}", i, n[i])] for i in range(3)]
    decode = []
    for i in range(3):
        decode.append([(f"d{i}", i, n[i] - 32)])
        decode += [[(f"d{i}", i, 1)] for _ in range(32)]
    portions = []
    for i in range(3):
        fed, j = 0, i
        while fed < n[i]:
            k = min(PORTIONS[j % len(PORTIONS)], n[i] - fed)
            portions.append([(f"p{i}", i, k)])
            fed, j = fed + k, j + 1
    # mixed: three live requests, portions of some beside single tokens of others; then the same
    # prompts again under new names, cut otherwise, in the pages the first wave gave back
    mixed = []
    for wave, cuts in enumerate(([40, 5, 17], [3, 64, 2])):
        fed = [0, 0, 0]
        key = lambda i: f"m{wave}{i}"
        step = 0
        while any(f < m for f, m in zip(fed, n)):
            entries = []
            for i in range(3):
                left = n[i] - fed[i]
                if left <= 0 or (step + i) % 5 == 4:
                    continue  # done, or left out of this step
                k = 1 if left <= 24 else min(left - 24, cuts[(i + step) % 3] if step % 3 else cuts[i])
                entries.append((key(i), i, k))
                fed[i] += k
            if entries:
                mixed.append(entries)
            step += 1
    return {"whole": whole, "decode": decode, "portions": portions, "mixed": mixed}


def _run(runner, prompts, plan):
    """Runs the steps (every token's logits wanted); returns {request key: (prompt, logits [n, V])}."""
    from from_scratch_inference_engine_amd.engine.context import StepEntry

    caches, fed, rows, which = {}, {}, {}, {}
    for step in plan:
        entries = []
        for key, i, k in step:
            if key not in caches:
                caches[key], fed[key], rows[key], which[key] = runner.manager.open(key), 0, [], i
            entries.append(StepEntry(caches[key], prompts[i][fed[key]:fed[key] + k], list(range(k))))
            fed[key] += k
        out = runner.step(entries).float().cpu()
        at = 0
        for key, i, k in step:
            rows[key].append(out[at:at + k])
            at += k
            if fed[key] == len(prompts[i]):
                runner.manager.close(caches[key])  # its pages go back; a later request takes them
        runner.manager.check_invariants()
    return {key: (which[key], torch.cat(r)) for key, r in rows.items()}


def test_float32_families_at_7b_widths(wide):
    from from_scratch_inference_engine_amd.engine.model import Model, Runner

    model = Model.from_pretrained(wide["dir"], dtype="float32")
    # 46 pages hold the three prompts together (21 + 19 + 5 pages) and one more: the second wave
    # of the mixed family can only run in the first wave's pages
    runner = Runner(model, page_size=16, num_pages=46, max_requests=4)
    worst = clear = rows = 0
    for family, plan in _plans().items():
        for key, (i, logits) in _run(runner, wide["prompts"], plan).items():
            ref = wide["ref"][i].numpy()
            assert logits.shape[0] == LENGTHS[i], f"{family} {key}: every position was asked for"
            c, r = helpers.assert_close_to_plain(logits.numpy(), ref, "float32", f"float32 {family} {key}")
            clear, rows = clear + c, rows + r
            worst = max(worst, float(np.abs(logits.numpy() - ref).max()))
    alloc = runner.manager.allocators[0]
    print(f"float32 at 7B widths, {LAYERS} layers: largest difference {worst:.3e}; argmax compared on {clear} of {rows} rows; "
          f"{alloc.pages_issued} pages handed out of a pool of {alloc.num_pages}")
    assert 2 * clear >= rows
    assert alloc.pages_issued > 4 * alloc.num_pages and len(alloc.pages_issued_again()) > alloc.num_pages * 3 // 4
    assert alloc.num_free == alloc.num_pages


def _assert_within_rounding(logits, ref, noise, what):
    diff = (logits - ref)
    worst, rms = diff.abs().max().item(), diff.pow(2).mean().sqrt().item()
    assert torch.isfinite(logits).all(), what
    assert worst <= 2.0 * noise[0], f"{what}: max|diff| {worst:.3e} against {noise[0]:.3e} from rounding alone"
    assert rms <= 1.5 * noise[1], f"{what}: rms diff {rms:.3e} against {noise[1]:.3e} from rounding alone"
    top2 = ref.topk(2, dim=-1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * worst
    assert torch.equal(logits.argmax(-1)[clear], ref.argmax(-1)[clear]), f"{what}: argmax differs on a clear row"
    return worst / noise[0], rms / noise[1]


def test_bfloat16_families_and_graph_batches_at_7b_widths(wide):
    from from_scratch_inference_engine_amd import ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Model, Runner

    model = Model.from_pretrained(wide["dir"], dtype="bfloat16")
    runner = Runner(model, page_size=16, num_pages=46, max_requests=4)
    ratios = []
    for family, plan in _plans().items():
        for key, (i, logits) in _run(runner, wide["prompts"], plan).items():
            ratios.append(_assert_within_rounding(logits, wide["ref"][i], wide["noise"][i], f"bfloat16 {family} {key}"))
    print(f"bfloat16 at 7B widths: difference / rounding noise, largest {max(r[0] for r in ratios):.2f} (max), "
          f"{max(r[1] for r in ratios):.2f} (rms)")
    del runner
    # decode batches of 32 to 160 rows: the engine's products up to 128 rows, the library's (chosen by
    # timing) beyond and for the small matrices, inside replayed graphs, with other work between the replays; the first eight requests against the plain model
    noise = max(n[0] for n in wide["noise"]), max(n[1] for n in wide["noise"])
    short, short_ref = wide["short"], wide["short_ref"]
    ops.enable_library_tuning(max_ms_per_candidate=5, iterations=2)
    own_rows = set()  # rows of the steps whose feed-forward products are the engine's own kernels
    real_swiglu, real_wide = ops.gemm_mfma_wide_swiglu, ops.gemm_mfma_wide
    ops.gemm_mfma_wide_swiglu = lambda x, w, **k: (own_rows.add(("gate/up", x.shape[0])), real_swiglu(x, w, **k))[1]
    ops.gemm_mfma_wide = lambda x, w, **k: (own_rows.add(("slices", x.shape[0])) if k.get("splits", 1) > 1 else None,
                                            real_wide(x, w, **k))[1]
    try:
        for batch in (32, 64, 80, 100, 128, 140):
            runner = Runner(model, page_size=16, num_pages=batch * 3 + 8, max_requests=batch)
            caches = [runner.manager.open(i) for i in range(batch)]
            runner.step([StepEntry(c, p[:-12], []) for c, p in zip(caches, short)])
            for t in range(12, 0, -1):
                out = runner.step([StepEntry(c, [p[-t]], [0]) for c, p in zip(caches, short)]).float().cpu()
                torch.cuda.synchronize()
                _ = (torch.randn(128, 128, device="cuda") @ torch.randn(128, 128, device="cuda")).sum().item()
                got = torch.stack([out[i] for i in range(8)])
                ref = torch.stack([short_ref[i][len(short[i]) - t] for i in range(8)])
                _assert_within_rounding(got, ref, noise, f"decode batch of {batch} through graphs, {t} from the end")
            assert runner.graphs.captures == 1 and runner.graphs.replays == 11
            del runner, caches
    finally:
        ops.disable_library_tuning()
        ops.gemm_mfma_wide_swiglu, ops.gemm_mfma_wide = real_swiglu, real_wide
    # 80, 100 and 128 requests run in graphs of 80, 112 and 128 rows, on the engine's kernels of five, seven
    # and eight tiles of rows over the fragment-ordered weights; 160 rows are the library's
    assert {("gate/up", r) for r in (80, 112, 128)} | {("slices", r) for r in (80, 112, 128)} <= own_rows, own_rows
    assert not any(rows > 128 for _, rows in own_rows), own_rows


def test_a_2048_token_step_with_the_librarys_timed_kernels_at_7b_widths(wide):
    """What the prefill measurement runs: one step of 2,048 tokens in bfloat16 with the library's
    kernels chosen by timing, against the plain logits at 24 places (the first and last tokens, the
    edges of pages and of the kernels' tiles, and places in between)."""
    from from_scratch_inference_engine_amd import ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Model, Runner

    long = wide["long"]
    model = Model.from_pretrained(wide["dir"], dtype="bfloat16")
    runner = Runner(model, page_size=16, num_pages=2048 // 16 + 40, max_requests=4)
    ops.enable_library_tuning(max_ms_per_candidate=5, iterations=2)
    try:
        for attempt in ("first (the library times its kernels)", "second (the kernels it kept)"):
            rc = runner.manager.open(attempt)
            got = runner.step([StepEntry(rc, long["ids"], long["rows"])]).float().cpu()
            runner.manager.close(rc)
            ratio = _assert_within_rounding(got, long["ref"], long["noise"], f"2,048-token step, {attempt}")
            print(f"2,048-token step, {attempt}: difference / rounding noise {ratio[0]:.2f} (max), {ratio[1]:.2f} (rms)")
    finally:
        ops.disable_library_tuning()
    # the same prompt in two portions of 1,024 beside a decoding request, without timing: same bound
    rc, other = runner.manager.open("portions"), runner.manager.open("other")
    short = wide["short"][0]
    runner.step([StepEntry(other, short[:-1], [])])
    rows = long["rows"]
    first = runner.step([StepEntry(rc, long["ids"][:1024], [r for r in rows if r < 1024])]).float().cpu()
    both = runner.step([StepEntry(other, short[-1:], [0]),
                        StepEntry(rc, long["ids"][1024:], [r - 1024 for r in rows if r >= 1024])]).float().cpu()
    _assert_within_rounding(torch.cat([first, both[1:]]), long["ref"], long["noise"], "2,048 tokens in two portions")
    _assert_within_rounding(both[:1], wide["short_ref"][0][-1:], long["noise"], "the token decoded beside a portion")


def test_engine_generates_the_plain_greedy_tokens_at_7b_widths(wide, monkeypatch):
    """tests/cpp/test_cuda_engine.cpp:45-79 at real widths: the engine (scheduler, one step ahead,
    graphs from the third step of a shape on, argmax over 152,064 logits on the device) in float32
    against greedy decoding by repeated whole forwards of the plain model.  A request is compared up
    to the first token whose plain lead over the runner-up is not clear."""
    from from_scratch_inference_engine_amd import Engine, SamplingParams
    from from_scratch_inference_engine_amd.engine import graphs
    from from_scratch_inference_engine_amd.engine.model import Model

    monkeypatch.setattr(graphs, "CAPTURE_AFTER", 3)  # the engine's own: eager steps, a capture, replays
    model = Model.from_pretrained(wide["dir"], dtype="float32")
    prompts = wide["short"][:3]
    for run_ahead in (True, False):
        engine = Engine(model, block_size=16, num_blocks=24, max_batch=4, max_tokens_per_step=64)
        engine.run_ahead = run_ahead
        got = engine.generate_batch(prompts, SamplingParams(temperature=0.0), max_tokens=12)
        compared = 0
        for out, (toks, leads) in zip(got, wide["greedy"]):
            assert len(out) == 12
            clear = next((i for i, lead in enumerate(leads) if lead <= 4 * helpers.F32_ATOL), len(leads))
            assert out[:clear] == toks[:clear], f"run_ahead={run_ahead}: {out} against plain {toks} (clear up to {clear})"
            compared += clear
        assert compared >= 24, f"only {compared} of 36 tokens had a clear plain choice"
        if run_ahead:
            assert engine.runner.graphs.replays > 0, "the decode steps were replayed from a graph"
        assert engine.free_blocks() == 24
    print(f"engine at 7B widths, float32: {compared} of 36 greedy tokens compared with plain")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_and_mixed_families_at_14b_widths(wide_14b, dtype):
    from from_scratch_inference_engine_amd.engine.model import Model, Runner

    model = Model.from_pretrained(wide_14b["dir"], dtype=dtype)
    runner = Runner(model, page_size=16, num_pages=46, max_requests=4)
    plans = _plans()
    worst = 0.0
    for family in ("decode", "mixed"):
        for key, (i, logits) in _run(runner, wide_14b["prompts"], plans[family]).items():
            ref = wide_14b["ref"][i]
            assert logits.shape[0] == LENGTHS[i]
            if dtype == "float32":
                helpers.assert_close_to_plain(logits.numpy(), ref.numpy(), "float32", f"14B widths float32 {family} {key}")
                worst = max(worst, float((logits - ref).abs().max()))
            else:
                r = _assert_within_rounding(logits, ref, wide_14b["noise"][i], f"14B widths bfloat16 {family} {key}")
                worst = max(worst, r[0])
    alloc = runner.manager.allocators[0]
    assert len(alloc.pages_issued_again()) > alloc.num_pages // 2 and alloc.num_free == alloc.num_pages
    print(f"{dtype} at 14B widths, {LAYERS_14B} layers: " +
          (f"largest difference {worst:.3e}" if dtype == "float32" else f"difference / rounding noise {worst:.2f}"))
