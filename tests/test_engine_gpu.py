"""Generation through the entry points on the GPU: greedy against the plain implementation,
long decoding, the first tokens of a sequence, the scheduler with a small pool, sampling."""

import json
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu


def plain_greedy(model_dir, prompt, n, eos=-1):
    cfg, w = plain.read_config(model_dir), plain.read_weights(model_dir)
    ids, out = list(prompt), []
    for _ in range(n):
        tok = plain.argmax(plain.forward(cfg, w, ids)[-1])
        out.append(tok)
        ids.append(tok)
        if tok == eos:
            break
    return out


@pytest.fixture(scope="module")
def llms(model_dirs):
    from from_scratch_inference_engine_amd import LLM

    return {(name, dtype): LLM(model_dirs[name], dtype=dtype, block_size=bs, num_blocks=64, max_batch=8)
            for name, bs in (("A", 4), ("B", 8)) for dtype in ("float32", "bfloat16")}


@pytest.mark.parametrize("name, lengths", [("A", [5, 11, 17]), ("B", [1, 7, 33])])
def test_greedy_generation_matches_plain_float32(llms, model_dirs, name, lengths):
    from from_scratch_inference_engine_amd import GenerationConfig

    llm = llms[(name, "float32")]
    vocab = helpers.TINY[name][0]["vocab_size"]
    prompts = [helpers.token_ids(vocab, n, 50 + n) for n in lengths]
    want = [plain_greedy(model_dirs[name], p, 16) for p in prompts]
    cfg = GenerationConfig(max_tokens=16, temperature=0.0)
    saved, llm.eos_id = llm.eos_id, -1
    try:
        assert [llm.generate_ids(p, cfg) for p in prompts] == want           # one at a time
        assert llm.generate_ids_batch(prompts, cfg) == want                   # batched by the scheduler
    finally:
        llm.eos_id = saved
    assert llm.engine.free_blocks() == 64


def test_llm_from_a_configuration_alone(tmp_path):
    """``LLM.from_config`` makes the weights on the device from a seed, without a folder: what it
    generates is what the folder written by ``write_random_model`` for that seed generates
    (float32 weights in the file, so that both hold the same values)."""
    from from_scratch_inference_engine_amd import LLM, GenerationConfig, load_config
    from from_scratch_inference_engine_amd.models import parse_config
    from from_scratch_inference_engine_amd.weights import write_random_model

    raw = dict(helpers.TINY["B"][0])  # (an untied head: what it generates depends on every weight)
    d = write_random_model(parse_config(raw), 21, tmp_path / "m", torch.float32)
    prompts = [helpers.token_ids(raw["vocab_size"], n, 70 + n) for n in (3, 9, 20)]
    cfg = GenerationConfig(max_tokens=12, temperature=0.0)
    want = [plain_greedy(d, p, 12) for p in prompts]
    for dtype in ("float32", "bfloat16"):
        direct = LLM.from_config(raw, 21, dtype=dtype, block_size=4, num_blocks=64)
        folder = LLM(d, dtype=dtype, block_size=4, num_blocks=64, eos_id=-1)
        got = direct.generate_ids_batch(prompts, cfg)
        assert got == folder.generate_ids_batch(prompts, cfg)
        if dtype == "float32":
            assert got == want
    with pytest.raises(RuntimeError, match="no tokenizer"):
        direct.generate("text")
    assert load_config(d).to_dict()["vocab_size"] == raw["vocab_size"]


def test_a_pool_as_large_as_the_free_memory(model_dirs, monkeypatch):
    """``num_blocks=0``: the pool takes nine tenths of the device's free memory less 2 GiB (here of a
    free memory that the test states), and generation from it is what a small pool gives."""
    from from_scratch_inference_engine_amd import LLM, GenerationConfig

    gib = 1 << 30
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (3 * gib, 288 * gib))
    llm = LLM(model_dirs["A"], dtype="float32", block_size=16, num_blocks=0)
    per_token = llm.model.cache_bytes_per_token()
    cfg = helpers.TINY_A
    layers, kv, hd = cfg["num_hidden_layers"], cfg["num_key_value_heads"], cfg["hidden_size"] // cfg["num_attention_heads"]
    assert per_token == layers * 2 * kv * hd * 4
    pages = llm.engine.runner.manager.allocators[0].num_pages
    assert pages == (int(3 * gib * 0.9) - 2 * gib) // (per_token * 16)
    monkeypatch.undo()
    prompt = helpers.token_ids(cfg["vocab_size"], 11, 5)
    small = LLM(model_dirs["A"], dtype="float32", block_size=16, num_blocks=8)
    gen = GenerationConfig(max_tokens=10, temperature=0.0)
    assert llm.generate_ids(prompt, gen) == small.generate_ids(prompt, gen) == plain_greedy(model_dirs["A"], prompt, 10)


def test_eos_from_the_folder_stops_generation(llms, model_dirs):
    from from_scratch_inference_engine_amd import GenerationConfig

    llm = llms[("B", "float32")]
    assert llm.eos_id == 7  # config.json of B
    prompt = helpers.token_ids(509, 9, 3)
    free = plain_greedy(model_dirs["B"], prompt, 12)
    llm.eos_id = free[4]
    try:
        got = llm.generate_ids(prompt, GenerationConfig(max_tokens=12))
    finally:
        llm.eos_id = 7
    stop = free.index(free[4])
    assert got == free[:stop + 1]  # the end-of-sequence token is kept


def test_bfloat16_generation_follows_plain_where_the_choice_is_clear(llms, model_dirs):
    """bfloat16 rounding may flip a near-tie; wherever the plain top-2 gap is wide the token is
    the plain one (teacher-forced on the plain continuation)."""
    from from_scratch_inference_engine_amd.engine.context import StepEntry

    llm = llms[("B", "bfloat16")]
    prompt = helpers.token_ids(509, 40, 4)
    cont = plain_greedy(model_dirs["B"], prompt, 24)
    ids = prompt + cont
    ref = plain.forward_dir(model_dirs["B"], ids)
    runner = llm.engine.runner
    rc = runner.manager.open("teacher")
    logits = runner.step([StepEntry(rc, ids, list(range(len(ids))))]).cpu()
    runner.manager.close(rc)
    top2 = ref.topk(2, dim=-1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * helpers.BF16_REL * ref.abs().max()
    assert clear.sum() >= 1
    assert torch.equal(logits.argmax(-1)[clear], ref.argmax(-1)[clear])
    helpers.assert_close_to_plain(logits.numpy(), ref.numpy(), "bfloat16", "teacher forced")


def test_long_decoding_and_first_tokens(llms, model_dirs):
    """250 positions of B, all but the first token decoded one by one: checks the first tokens of
    a sequence (positions 0, 1, 2 at every page offset) and a long run over many pages."""
    from from_scratch_inference_engine_amd.engine.context import StepEntry

    ids = helpers.token_ids(509, 250, 5)
    ref = plain.forward_dir(model_dirs["B"], ids).numpy()
    for dtype in ("float32", "bfloat16"):
        runner = llms[("B", dtype)].engine.runner
        rc = runner.manager.open("long")
        rows = [runner.step([StepEntry(rc, ids[t:t + 1], [0])]) for t in range(len(ids))]
        runner.manager.close(rc)
        got = torch.cat(rows).cpu().numpy()
        helpers.assert_close_to_plain(got[:3], ref[:3], dtype, f"first tokens {dtype}")
        helpers.assert_close_to_plain(got, ref, dtype, f"long decoding {dtype}")


def test_small_pool_preempts_and_still_matches(model_dirs):
    """tests/cpp/test_engine.cpp:103-128 on the GPU: pages run out, the youngest request is
    preempted and recomputed; outputs equal the plain greedy continuation."""
    from from_scratch_inference_engine_amd import Engine, SamplingParams, SeqStatus, load_model

    model = load_model(model_dirs["A"], dtype="float32")
    engine = Engine(model, block_size=4, num_blocks=6, max_batch=4, max_tokens_per_step=8)
    prompts = [helpers.token_ids(256, n, 70 + n) for n in (4, 4, 7, 3)]
    ids = [engine.add_request(p, SamplingParams(temperature=0.0), max_tokens=9) for p in prompts]
    steps = 0
    while engine.has_work():
        engine.step()
        steps += 1
        assert steps < 400
    assert engine.preemptions() > 0
    assert all(engine.status(i) == SeqStatus.Finished for i in ids)
    for i, p in zip(ids, prompts):
        assert engine.output(i) == plain_greedy(model_dirs["A"], p, 9)
    assert engine.free_blocks() == 6
    with pytest.raises(ValueError, match="never run"):
        engine.add_request(list(range(20)), max_tokens=8)
    with pytest.raises(IndexError, match="vocabulary"):
        engine.add_request([1, 256], max_tokens=2)


def test_a_preempted_request_draws_the_same_samples_again(model_dirs):
    """Temperature 0.7 in a pool so small that requests are preempted and recomputed: every
    request's tokens are those of a pool that never preempts.  A draw belongs to (seed, request,
    token index), so the recomputed request meets the same uniform numbers at the same places; a
    generator shared by the batch, or one that counts draws, would give other tokens here."""
    from from_scratch_inference_engine_amd import Engine, SamplingParams, SeqStatus, load_model

    model = load_model(model_dirs["A"], dtype="float32")
    prompts = [helpers.token_ids(256, n, 70 + n) for n in (4, 4, 7, 3)]
    params = SamplingParams(temperature=0.7)

    def run(num_blocks, seed=3):
        engine = Engine(model, block_size=4, num_blocks=num_blocks, seed=seed, max_batch=4, max_tokens_per_step=8)
        ids = [engine.add_request(p, params, max_tokens=9) for p in prompts]
        steps = 0
        while engine.has_work():
            engine.step()
            steps += 1
            assert steps < 400
        assert all(engine.status(i) == SeqStatus.Finished for i in ids)
        assert engine.free_blocks() == num_blocks
        return [engine.output(i) for i in ids], engine.preemptions()

    roomy, none = run(64)
    tight, some = run(6)
    assert none == 0 and some > 0
    assert tight == roomy
    assert run(64, seed=4)[0] != roomy                      # the draws do depend on the seed
    greedy = Engine(model, block_size=4, num_blocks=64, max_batch=4, max_tokens_per_step=8)
    assert greedy.generate_batch(prompts, SamplingParams(temperature=0.0), max_tokens=9) != roomy  # and are draws


def test_temperature_sampling_is_reproducible_and_independent_of_the_batch(llms):
    """Two engines with the same seed: all requests at once in one, one at a time in the other.
    Draws belong to (seed, request, token index), so the outputs are the same."""
    from from_scratch_inference_engine_amd import Engine, SamplingParams

    model = llms[("B", "float32")].model
    prompts = [helpers.token_ids(509, n, 80 + n) for n in (1, 7, 33, 64, 90)]
    params = SamplingParams(temperature=0.7)

    def engine(seed):
        return Engine(model, block_size=8, num_blocks=64, seed=seed, max_batch=8, max_tokens_per_step=48,
                      prefill_chunk=16)

    together = engine(5).generate_batch(prompts, params, max_tokens=12)
    one = engine(5)
    alone = [one.generate(p, params, max_tokens=12) for p in prompts]
    assert together == alone
    assert engine(6).generate_batch(prompts, params, max_tokens=12) != together
    greedy = engine(5).generate_batch(prompts, SamplingParams(temperature=0.0), max_tokens=12)
    assert greedy != together
    # the same mixed, chunked run, greedy: the plain continuation of every prompt
    assert greedy == [plain_greedy(llms[("B", "float32")]._model_dir, p, 12) for p in prompts]


def test_command_line_generate(model_dirs):
    prompt = helpers.token_ids(256, 6, 9)
    cmd = [sys.executable, "-m", "from_scratch_inference_engine_amd", "generate", "--model-dir", str(model_dirs["A"]),
           "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompt)), "--max-tokens", "8", "--block-size", "4",
           "--num-blocks", "32", "--json"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(helpers.ROOT))
    assert proc.returncode == 0, proc.stderr[-3000:]
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    assert out["outputs"] == [plain_greedy(model_dirs["A"], prompt, 8)]


def test_command_line_generate_from_a_configuration(tmp_path):
    """--config FILE --random-weights SEED: no model folder; the same tokens as the folder that
    random-model writes for that seed."""
    from from_scratch_inference_engine_amd.models import parse_config
    from from_scratch_inference_engine_amd.weights import write_random_model

    raw = dict(helpers.TINY["B"][0])
    (tmp_path / "cfg.json").write_text(json.dumps(raw))
    d = write_random_model(parse_config(raw), 33, tmp_path / "m", torch.float32)
    prompt = helpers.token_ids(raw["vocab_size"], 7, 19)
    cmd = [sys.executable, "-m", "from_scratch_inference_engine_amd", "generate", "--config", str(tmp_path / "cfg.json"),
           "--random-weights", "33", "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompt)), "--max-tokens", "6",
           "--block-size", "8", "--num-blocks", "16", "--json"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(helpers.ROOT))
    assert proc.returncode == 0, proc.stderr[-3000:]
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    assert out["outputs"] == [plain_greedy(d, prompt, 6)]
    bad = subprocess.run(cmd[:5] + cmd[7:], capture_output=True, text=True, timeout=300, cwd=str(helpers.ROOT))
    assert bad.returncode != 0 and "go together" in bad.stderr


def test_graft_entry_smoke():
    import __graft_entry__ as entry

    entry.smoke()


def test_bench_prints_its_line():
    """bench.py as it is run for the record, at a small shape (two layers of 896 / 4864): the library's
    kernels chosen by timing, prefill, decode at batch 8, 1 and 64 through the engine, the time of each
    class of kernels; one JSON line with the fields of the contract.  More than one GPU: one line, exit 2."""
    cmd = [sys.executable, "bench.py", "--shape", "0.5b", "--layers", "2", "--steps", "8", "--warmup", "4"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(helpers.ROOT))
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = proc.stdout.strip().splitlines()
    assert len(lines) == 1, lines
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points", "kernels"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 8 and rec["warmup"] == 4 and rec["dtype"] == "bf16"
    assert rec["value"] > 0 and abs(rec["value"] - 8 / (rec["ms_per_step"] * 1e-3)) <= 1e-6 * rec["value"]
    assert len(rec["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in rec["config"].values())
    assert rec["config"]["layers"] == 2 and rec["config"]["layers_of_config"] == 24
    assert rec["config"]["streamed_weight_copies"] is True and rec["config"]["library_gemm_tuning"] is True
    assert rec["prefill"]["tokens"] == 2048 and 0 < rec["prefill"]["frac"] < 1
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["peak"] == 8000.0 and 0 < rec["roofline"]["frac"] < 1
    assert set(rec["points"]) == {"decode_b1", "decode_b64"} == set(rec["points_roofline_frac"])
    assert all(0 < f < 1 for f in rec["points_roofline_frac"].values())
    assert {"attention", "qkv", "gate_up", "down", "o", "norms", "lm_head"} <= set(rec["kernels"])
    assert all(v["ms"] > 0 and v["launches"] > 0 for v in rec["kernels"].values())
    two = subprocess.run(cmd[:2] + ["--gpus", "2"], capture_output=True, text=True, timeout=120, cwd=str(helpers.ROOT))
    assert two.returncode == 2 and len(two.stdout.strip().splitlines()) == 1


def test_graph_replays_equal_eager_steps(model_dirs):
    """Decode steps run as replayed graphs.  Two runners over the same model, one with graphs and
    one without, decode the same 20 requests (more rows than the engine's own small-matrix kernel
    takes, so the library product is inside the graph too) for several steps, with other eager
    work and synchronisations between the replays; every step's logits must agree, and contexts
    that grow across a bucket edge must capture again and still agree."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    model = load_model(model_dirs["B"], dtype="bfloat16")
    runners = [Runner(model, page_size=4, num_pages=640, max_requests=32, use_graphs=g) for g in (True, False)]
    prompts = [helpers.token_ids(509, 3 + 5 * i, 300 + i) for i in range(20)]
    caches = [[r.manager.open(i) for i in range(20)] for r in runners]
    for r, cs in zip(runners, caches):
        r.step([StepEntry(c, p, []) for c, p in zip(cs, prompts)])
    feed = [helpers.token_ids(509, 40, 400 + i) for i in range(20)]
    for t in range(40):
        outs = []
        for r, cs in zip(runners, caches):
            outs.append(r.step([StepEntry(c, [feed[i][t]], [0]) for i, c in enumerate(cs)]).float().cpu())
            torch.cuda.synchronize()
            _ = (torch.randn(64, 64, device="cuda") @ torch.randn(64, 64, device="cuda")).sum().item()  # eager work between replays
        assert torch.equal(outs[0], outs[1]), f"decode step {t}"
    g = runners[0].graphs
    assert g.captures >= 2 and g.replays >= 30
    # a step that is not a plain decode step does not go through a graph
    before = g.captures + g.replays
    runners[0].step([StepEntry(caches[0][0], [1, 2], [1])])
    assert g.captures + g.replays == before


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_that_shrinks_decodes_through_graphs_of_padded_sizes(model_dirs, dtype):
    """Seven requests decode together and end one after the other.  Graphs are captured for 8, 4,
    2 and 1 rows only (the rows that fill a batch up read and write the spare page); what every
    batch size returns for the real requests is what the eager runner returns (which runs the
    unpadded batch), agrees with the plain model, and a request that comes later and is given the pages of one that ended
    is not disturbed by what the filler rows wrote."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.graphs import padded_rows
    from from_scratch_inference_engine_amd.engine.model import Runner

    assert [padded_rows(n) for n in (1, 2, 3, 4, 5, 8, 9, 16, 17, 33, 64, 65, 100, 113, 129, 130)] == \
        [1, 2, 4, 4, 8, 8, 16, 16, 32, 48, 64, 80, 112, 128, 160, 160]
    model = load_model(model_dirs["A"], dtype=dtype)
    vocab = plain.read_config(model_dirs["A"])["vocab_size"]
    seqs = [helpers.token_ids(vocab, 30 + 3 * i, 900 + i) for i in range(7)]
    late = helpers.token_ids(vocab, 20, 950)
    ref = [plain.forward_dir(model_dirs["A"], ids).numpy() for ids in seqs + [late]]
    runners = [Runner(model, page_size=4, num_pages=96, max_requests=8, use_graphs=g) for g in (True, False)]
    caches = [[r.manager.open(i) for i in range(7)] for r in runners]
    n_pre = [len(ids) - (3 + 2 * i) for i, ids in enumerate(seqs)]  # request i decodes 3 + 2 i tokens, then ends
    for r, cs in zip(runners, caches):
        r.step([StepEntry(c, ids[:n], []) for c, ids, n in zip(cs, seqs, n_pre)])
    live = list(range(7))
    t = 0
    while live:
        outs = []
        for r, cs in zip(runners, caches):
            outs.append(r.step([StepEntry(cs[i], [seqs[i][n_pre[i] + t]], [0]) for i in live]).float().cpu())
        helpers.assert_close_to_plain(outs[0].numpy(), outs[1].numpy(), dtype, f"step {t} with {len(live)} requests, graphs against eager")
        for row, i in enumerate(live):
            helpers.assert_close_to_plain(outs[0][row:row + 1].numpy(), ref[i][n_pre[i] + t:n_pre[i] + t + 1], dtype,
                                          f"step {t}, request {i} in a batch of {len(live)}")
        t += 1
        for i in [i for i in live if n_pre[i] + t == len(seqs[i])]:
            live.remove(i)
            for r, cs in zip(runners, caches):
                r.manager.close(cs[i])
    g = runners[0].graphs
    assert g.captures <= 5 and g.replays >= t - 5, (g.captures, g.replays)
    # the pages of the ended requests, handed out again
    for r in runners:
        c = r.manager.open("late")
        out = r.step([StepEntry(c, late[:-2], [])])
        for j in (2, 1):
            out = r.step([StepEntry(c, [late[-j]], [0])]).float().cpu().numpy()
            helpers.assert_close_to_plain(out, ref[7][len(late) - j:len(late) - j + 1], dtype, f"late request, token -{j}")


def test_a_shape_is_captured_the_third_time_it_comes(model_dirs, monkeypatch):
    """With the engine's own threshold the first two decode steps of a shape run eagerly, the
    third captures its graph and later ones replay it; all of them agree with the plain model."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine import graphs
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    monkeypatch.setattr(graphs, "CAPTURE_AFTER", 3)
    model = load_model(model_dirs["B"], dtype="bfloat16")
    runner = Runner(model, page_size=8, num_pages=32, max_requests=2)
    assert runner.graphs.capture_after == 3
    vocab = plain.read_config(model_dirs["B"])["vocab_size"]
    ids = helpers.token_ids(vocab, 30, 960)
    ref = plain.forward_dir(model_dirs["B"], ids).numpy()
    cache = runner.manager.open("a")
    runner.step([StepEntry(cache, ids[:24], [])])
    seen = []
    for t in range(24, 30):
        out = runner.step([StepEntry(cache, [ids[t]], [0])]).float().cpu().numpy()
        helpers.assert_close_to_plain(out, ref[t:t + 1], "bfloat16", f"token {t}")
        seen.append((runner.graphs.captures, runner.graphs.replays))
    assert seen == [(0, 0), (0, 0), (1, 0), (1, 1), (1, 2), (1, 3)]


@pytest.mark.parametrize("name", ["A", "B"])
def test_decoding_with_partial_sums_in_the_residual_stream(model_dirs, name, monkeypatch):
    """The tiny models are too narrow for the projections to cut K by themselves, so the cut is
    forced: the output and down projections then leave float32 partial sums that the next norm
    (and the model's last one, on chosen rows) adds up.  Decoded in a batch, eagerly and through
    graphs, against the plain implementation."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner
    from from_scratch_inference_engine_amd.parts.linear import Linear

    used = []

    def two_if_it_fits(self, m):
        fits = -(-(-(-self.in_features // 2)) // 64) * 64 < self.in_features
        used.append(fits)
        return 2 if fits else 1

    monkeypatch.setattr(Linear, "residual_splits", two_if_it_fits)
    model = load_model(model_dirs[name], dtype="bfloat16")
    assert model.partial_sums_ok
    vocab = plain.read_config(model_dirs[name])["vocab_size"]
    seqs = [helpers.token_ids(vocab, 21 + 9 * i, 700 + i) for i in range(3)]
    ref = [plain.forward_dir(model_dirs[name], ids).numpy() for ids in seqs]
    for graphs in (False, True):
        runner = Runner(model, page_size=4, num_pages=64, max_requests=4, use_graphs=graphs)
        caches = [runner.manager.open(i) for i in range(3)]
        n_pre = [len(ids) - 8 for ids in seqs]
        runner.step([StepEntry(c, ids[:n], []) for c, ids, n in zip(caches, seqs, n_pre)])
        for t in range(8):
            out = runner.step([StepEntry(c, [ids[n + t]], [0]) for c, ids, n in zip(caches, seqs, n_pre)]).float().cpu()
            for i in range(3):
                helpers.assert_close_to_plain(out[i:i + 1].numpy(), ref[i][n_pre[i] + t:n_pre[i] + t + 1], "bfloat16",
                                              f"{name} graphs={graphs} request {i} token {t}")
    assert any(used)


WIDE = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 1024, "num_hidden_layers": 2, "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 128,
    "intermediate_size": 1536, "vocab_size": 331, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 512,
}


def test_batches_of_17_to_64_rows_share_x_through_lds(tmp_path):
    """A model wide enough (inner sizes that are multiples of 128 and at least 1,024) that steps
    of 17 to 64 rows take the kernel that shares x through LDS: the output and down projections
    as partial sums for the next norm, the logits whole.  20 requests decode together, eagerly
    and through graphs, and a 40-token portion runs beside 3 decoded tokens."""
    from from_scratch_inference_engine_amd import load_model, ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    d = helpers.make_model_dir(tmp_path / "wide", WIDE, seed=9)
    model = load_model(d, dtype="bfloat16")
    calls = []
    real = ops.gemm_mfma_wide

    def counted(x, w, splits=1, **kw):
        calls.append((x.shape[0], splits))
        return real(x, w, splits=splits, **kw)

    ops.gemm_mfma_wide = counted
    real_rope, summed = ops.rope_kv_write, []

    def rope_counted(qkv, *a, parts=None, **kw):
        summed.append((qkv.shape[0], parts is not None))
        return real_rope(qkv, *a, parts=parts, **kw)

    ops.rope_kv_write = rope_counted
    try:
        seqs = [helpers.token_ids(331, 9 + i, 900 + i) for i in range(20)]
        long = helpers.token_ids(331, 60, 950)
        ref = [plain.forward_dir(d, ids).numpy() for ids in seqs[:6]]
        ref_long = plain.forward_dir(d, long).numpy()
        for graphs in (False, True):
            runner = Runner(model, page_size=16, num_pages=64, max_requests=24, use_graphs=graphs)
            caches = [runner.manager.open(i) for i in range(20)]
            n_pre = [len(ids) - 4 for ids in seqs]
            runner.step([StepEntry(c, ids[:n], []) for c, ids, n in zip(caches, seqs, n_pre)])
            for t in range(4):
                out = runner.step([StepEntry(c, [ids[n + t]], [0]) for c, ids, n in zip(caches, seqs, n_pre)]).float().cpu()
                for i in range(6):
                    helpers.assert_close_to_plain(out[i:i + 1].numpy(), ref[i][n_pre[i] + t:n_pre[i] + t + 1], "bfloat16",
                                                  f"graphs={graphs} request {i} token {t}")
            for c in caches[3:]:
                runner.manager.close(c)
            # a portion of 40 tokens beside three decoded tokens: 43 rows in one step
            lc = runner.manager.open("long")
            runner.step([StepEntry(lc, long[:20], [])])
            out = runner.step([StepEntry(lc, long[20:], list(range(40)))]).float().cpu()
            helpers.assert_close_to_plain(out.numpy(), ref_long[20:], "bfloat16", f"graphs={graphs} portion of 40")
    finally:
        ops.gemm_mfma_wide = real
        ops.rope_kv_write = real_rope
    # q/k/v of 17 to 64 rows come as partial sums that the rotation adds up; longer steps whole
    assert {m for m, parts in summed if parts} >= {20, 40} and all(parts == (16 < m <= 64) for m, parts in summed), summed
    rows = {m for m, _ in calls}
    assert 20 in rows and 40 in rows, rows                      # decode batch and the portion
    used = {s for _, s in calls}
    assert 1 in used and len(used) > 1 and all(1 <= s <= 16 for s in used), calls  # logits whole, projections in slices


def test_steps_of_one_token_a_request_finish_qkv_inside_attention(tmp_path, monkeypatch):
    """Steps in which every request has one token hand the q/k/v product's partial sums to the
    attention kernel, which adds them up, rotates, scores the new key and writes the cache itself:
    1, 3 and 20 requests decoding, eagerly and through graphs, against the plain model; the tokens
    such steps wrote are then read by a portion of several tokens; and with the switch off the same
    steps give the same logits up to rounding through the kernels that do these one after the other."""
    from from_scratch_inference_engine_amd import load_model, ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner
    from from_scratch_inference_engine_amd.parts.attention import GQAttention

    d = helpers.make_model_dir(tmp_path / "wide", WIDE, seed=13)
    model = load_model(d, dtype="bfloat16")
    fused, apart = [], []
    real_qkv, real_rope, real_project = ops.attention_mfma_qkv, ops.rope_kv_write, ops.gemm_mfma_skinny_rope
    monkeypatch.setattr(ops, "attention_mfma_qkv", lambda sums, *a, **k: (fused.append(sums.shape[:2]), real_qkv(sums, *a, **k))[1])
    monkeypatch.setattr(ops, "rope_kv_write", lambda qkv, *a, **k: (apart.append(qkv.shape[0]), real_rope(qkv, *a, **k))[1])
    monkeypatch.setattr(ops, "gemm_mfma_skinny_rope", lambda x, *a, **k: (apart.append(x.shape[0]), real_project(x, *a, **k))[1])
    seqs = [helpers.token_ids(331, 40 + 3 * i, 700 + i) for i in range(20)]
    ref = [plain.forward_dir(d, ids).numpy() for ids in seqs[:4]]
    logits = {}
    for on in (True, False):
        monkeypatch.setattr(GQAttention, "finish_qkv_in_attention", on)
        for graphs in (False, True):
            for live in (1, 3, 20):
                runner = Runner(model, page_size=16, num_pages=160, max_requests=24, use_graphs=graphs)
                caches = [runner.manager.open(i) for i in range(live)]
                n_pre = [len(ids) - 9 for ids in seqs[:live]]
                runner.step([StepEntry(c, ids[:n], []) for c, ids, n in zip(caches, seqs, n_pre)])
                fused.clear(), apart.clear()
                for t in range(5):  # five tokens one by one ...
                    out = runner.step([StepEntry(c, [ids[n + t]], [0]) for c, ids, n in zip(caches, seqs, n_pre)]).float().cpu()
                    logits[(on, graphs, live, t)] = out
                    for i in range(min(live, 4)):
                        helpers.assert_close_to_plain(out[i:i + 1].numpy(), ref[i][n_pre[i] + t:n_pre[i] + t + 1], "bfloat16",
                                                      f"in attention={on} graphs={graphs} {live} live, request {i} token {t}")
                if not graphs:
                    assert (len(fused) == 5 * 2 and not apart) if on else (len(apart) == 5 * 2 and not fused), (on, fused, apart)
                    assert all(shape[1] == live and shape[0] >= 2 for shape in fused), fused
                # ... then the last four of the first request together: they read what those steps wrote
                out = runner.step([StepEntry(caches[0], seqs[0][n_pre[0] + 5:], [0, 1, 2, 3])]).float().cpu()
                helpers.assert_close_to_plain(out.numpy(), ref[0][n_pre[0] + 5:], "bfloat16",
                                              f"in attention={on} graphs={graphs} {live} live: four tokens after the decoded ones")
    for (on, graphs, live, t), out in logits.items():
        if on:
            other = logits[(False, graphs, live, t)]
            assert (out - other).abs().max() <= 2.0 ** -6 * other.abs().max(), (graphs, live, t)


def test_decoding_from_fragment_ordered_copies(tmp_path, monkeypatch):
    """With the size from which a weight is kept a second time, in the order of the matrix
    instruction's fragments, set to zero, the small wide model keeps copies of every matrix whose
    inner size the kernel takes (q/k/v, output, gate/up, down, the head of 331 rows, which ends inside
    a block of 16), and steps of up to 64 rows read them (q/k/v from 17 rows on; with fewer its product
    has the rotation in its epilogue and reads rows): 1, 3 and 20 requests decoding, eagerly and
    through graphs, and a portion of 40 tokens beside 3 decoded ones, against the plain model.  A
    weight that is set anew drops its copy."""
    from from_scratch_inference_engine_amd import load_model, ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner
    from from_scratch_inference_engine_amd.parts.linear import Linear

    d = helpers.make_model_dir(tmp_path / "wide", WIDE, seed=11)
    plain_model = load_model(d, dtype="bfloat16")
    assert plain_model.spec.lm_head.linear.streamed is None  # 0.7 MB: far below the size that is copied
    monkeypatch.setattr(Linear, "streamed_copy_from", 0)
    from from_scratch_inference_engine_amd.engine.model import Model
    without = Model.from_pretrained(d, dtype="bfloat16", weight_copies=False)
    assert without.spec.lm_head.linear.streamed is None and Linear.streamed_copy_from == 0
    del without
    model = load_model(d, dtype="bfloat16")
    block = model.spec.layers[0]
    copies = [model.spec.lm_head.linear, block.mixer.o, block.mixer.qkv, block.ffn.gate_up, block.ffn.down]
    assert all(isinstance(c.streamed, ops.FragmentOrdered) and c.streamed.shape == tuple(c.weight.shape) for c in copies)
    seen = []
    real, real_swiglu = ops.gemm_mfma_wide, ops.gemm_mfma_wide_swiglu

    def counted(x, w, **kw):
        seen.append(("plain", x.shape[0], isinstance(w, ops.FragmentOrdered)))
        return real(x, w, **kw)

    def counted_swiglu(x, w, **kw):
        seen.append(("swiglu", x.shape[0], isinstance(w, ops.FragmentOrdered)))
        return real_swiglu(x, w, **kw)

    monkeypatch.setattr(ops, "gemm_mfma_wide", counted)
    monkeypatch.setattr(ops, "gemm_mfma_wide_swiglu", counted_swiglu)
    seqs = [helpers.token_ids(331, 9 + i, 400 + i) for i in range(20)]
    long = helpers.token_ids(331, 60, 450)
    ref = [plain.forward_dir(d, ids).numpy() for ids in seqs[:4]]
    ref_long = plain.forward_dir(d, long).numpy()
    for graphs in (False, True):
        for live in (1, 3, 20):
            runner = Runner(model, page_size=16, num_pages=64, max_requests=24, use_graphs=graphs)
            caches = [runner.manager.open(i) for i in range(live)]
            n_pre = [len(ids) - 5 for ids in seqs[:live]]  # four tokens decoded here, the fifth beside the portion
            runner.step([StepEntry(c, ids[:n], []) for c, ids, n in zip(caches, seqs, n_pre)])
            for t in range(4):
                out = runner.step([StepEntry(c, [ids[n + t]], [0]) for c, ids, n in zip(caches, seqs, n_pre)]).float().cpu()
                for i in range(min(live, 4)):
                    helpers.assert_close_to_plain(out[i:i + 1].numpy(), ref[i][n_pre[i] + t:n_pre[i] + t + 1], "bfloat16",
                                                  f"graphs={graphs} {live} live, request {i} token {t}")
        for c in caches[3:]:
            runner.manager.close(c)
        lc = runner.manager.open("long")
        runner.step([StepEntry(lc, long[:20], [])])
        entries = [StepEntry(lc, long[20:], list(range(40)))]
        entries += [StepEntry(c, [ids[n + 4]], [0]) for c, ids, n in zip(caches[:3], seqs, n_pre)]
        out = runner.step(entries).float().cpu()
        helpers.assert_close_to_plain(out[:40].numpy(), ref_long[20:], "bfloat16", f"graphs={graphs} portion of 40")
        for i in range(3):
            helpers.assert_close_to_plain(out[40 + i:41 + i].numpy(), ref[i][n_pre[i] + 4:n_pre[i] + 5], "bfloat16",
                                          f"graphs={graphs} request {i} beside the portion")
    assert seen and all(frag for _, _, frag in seen), seen
    assert {m for kind, m, _ in seen if kind == "swiglu"} >= {1, 3, 20, 43}
    assert {m for kind, m, _ in seen if kind == "plain"} >= {1, 3, 20, 43}
    lin = model.spec.lm_head.linear
    lin.weight = lin.weight.clone()
    assert lin.streamed is None
    lin.prepare()
    assert lin.streamed is not None
    monkeypatch.setattr(Linear, "streamed_copy_reserve", 1.0)  # no copy may leave that much of the device free
    lin.prepare()
    assert lin.streamed is None


def test_a_cache_that_does_not_fit_beside_the_weight_copies_drops_them(tmp_path, monkeypatch):
    """The second copies of the large weights are made when the model is loaded, before anybody
    knows how large the cache will be.  If the pools then do not fit, the copies go and the pools
    are asked for again; the model decodes from rows and gives the same tokens.  (The first request
    for the pools is made to fail from the host: no memory is exhausted here.)"""
    import warnings

    from from_scratch_inference_engine_amd import LLM, Engine, GenerationConfig, SamplingParams
    from from_scratch_inference_engine_amd.cache import storage as storage_module
    from from_scratch_inference_engine_amd.parts.linear import Linear

    monkeypatch.setattr(Linear, "streamed_copy_from", 0)  # every matrix of the tiny model has a copy
    cfg = dict(helpers.TINY_B, hidden_size=256, num_attention_heads=8, head_dim=32, intermediate_size=384)
    d = helpers.make_model_dir(tmp_path / "m", cfg, seed=5)
    llm = LLM(d, dtype="bfloat16", block_size=8, num_blocks=32, max_batch=4, eos_id=-1)
    mixer = llm.model.spec.layers[0].mixer
    assert mixer.o.streamed is not None and llm.model.spec.lm_head.linear.streamed is not None
    prompts = [helpers.token_ids(509, n, 1600 + n) for n in (5, 19)]
    gen = GenerationConfig(max_tokens=10, temperature=0.0)
    with_copies = llm.generate_ids_batch(prompts, gen)

    real_init = storage_module.CacheStorage.__init__
    failed = []

    def init(self, *a, **k):
        if not failed:
            failed.append(1)
            raise torch.cuda.OutOfMemoryError("(the test says so)")
        real_init(self, *a, **k)

    monkeypatch.setattr(storage_module.CacheStorage, "__init__", init)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        engine = Engine(llm.model, block_size=8, num_blocks=32, max_batch=4)
    assert failed and any("copies dropped" in str(w.message) for w in caught)
    assert all(lin.streamed is None for block in llm.model.spec.layers
               for lin in (block.mixer.qkv, block.mixer.o, block.ffn.gate_up, block.ffn.down))
    assert llm.model.spec.lm_head.linear.streamed is None
    without = engine.generate_batch(prompts, SamplingParams(temperature=0.0), max_tokens=10)
    assert without == with_copies  # (the products on the copy and on rows give the same bits)


def test_prefill_with_the_library_kernel_selection(model_dirs):
    """With tuning on, a prompt portion of a multiple of 256 rows, and a decode batch of a multiple
    of 16, let torch time the library's candidates for their products; whatever it picks, the
    logits stay those of the plain model."""
    from from_scratch_inference_engine_amd import load_model, ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    vocab = plain.read_config(model_dirs["B"])["vocab_size"]
    ids = helpers.token_ids(vocab, 256, 810)
    ref = plain.forward_dir(model_dirs["B"], ids).numpy()
    ops.enable_library_tuning(max_ms_per_candidate=5, iterations=2)
    try:
        assert ops.library_tuning_enabled()
        runner = Runner(load_model(model_dirs["B"], dtype="bfloat16"), page_size=16, num_pages=32, max_requests=2)
        out = runner.step([StepEntry(runner.manager.open("a"), ids, list(range(256)))]).float().cpu().numpy()
        # a decode batch of 32: its library products are timed in the eager run before the capture,
        # the captured graph then replays the chosen kernels
        runner = Runner(load_model(model_dirs["B"], dtype="bfloat16"), page_size=16, num_pages=80, max_requests=32)
        seqs = [helpers.token_ids(vocab, 6 + i % 5, 820 + i) for i in range(32)]
        refs = [plain.forward_dir(model_dirs["B"], s_).numpy() for s_ in seqs[:5]]
        caches = [runner.manager.open(i) for i in range(32)]
        runner.step([StepEntry(c, s_[:-3], []) for c, s_ in zip(caches, seqs)])
        decoded = []
        for t in range(3, 0, -1):
            decoded.append(runner.step([StepEntry(c, [s_[-t]], [0]) for c, s_ in zip(caches, seqs)]).float().cpu().numpy())
        assert runner.graphs.captures == 1 and runner.graphs.replays == 2
        # with the timing on, a step of 107 tokens is filled up to 128 with the tokens of a request
        # that does not exist: what the real requests get does not change, nor what they decode next
        from from_scratch_inference_engine_amd.engine.context import padded_tokens
        assert padded_tokens(70 + 37) == 128
        runner = Runner(load_model(model_dirs["B"], dtype="bfloat16"), page_size=8, num_pages=40, max_requests=3,
                        fill_rows=padded_tokens)
        pair = [helpers.token_ids(vocab, 71, 870), helpers.token_ids(vocab, 38, 871)]
        pair_ref = [plain.forward_dir(model_dirs["B"], s_).numpy() for s_ in pair]
        pc = [runner.manager.open(i) for i in range(2)]
        filled = runner.step([StepEntry(c, s_[:-1], [len(s_) - 2]) for c, s_ in zip(pc, pair)]).float().cpu().numpy()
        after = runner.step([StepEntry(c, [s_[-1]], [0]) for c, s_ in zip(pc, pair)]).float().cpu().numpy()
    finally:
        ops.disable_library_tuning()
    for i, s_ in enumerate(pair):
        helpers.assert_close_to_plain(filled[i:i + 1], pair_ref[i][len(s_) - 2:len(s_) - 1], "bfloat16",
                                      f"filled-up step, request {i}")
        helpers.assert_close_to_plain(after[i:i + 1], pair_ref[i][len(s_) - 1:], "bfloat16",
                                      f"decoding after a filled-up step, request {i}")
    helpers.assert_close_to_plain(out, ref, "bfloat16", "prefill of 256 rows with library tuning")
    for i in range(5):
        for j in range(3):
            helpers.assert_close_to_plain(decoded[j][i:i + 1], refs[i][len(seqs[i]) - 3 + j:len(seqs[i]) - 2 + j], "bfloat16",
                                          f"decode batch of 32 with library tuning, request {i} token {j}")


def test_a_dropped_runner_frees_its_graphs_at_once(model_dirs):
    """A runner and its graphs form no reference cycle: dropping the runner destroys the captured
    graphs then, by reference count, not when the collector of cycles next runs.  (A collector run
    in the middle of another runner's capture would free their memory there, which ends the
    process.)"""
    import gc
    import weakref

    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    model = load_model(model_dirs["A"], dtype="bfloat16")
    gc.collect()
    gc.disable()
    try:
        runner = Runner(model, page_size=4, num_pages=32, max_requests=2)
        cache = runner.manager.open("a")
        runner.step([StepEntry(cache, [1, 2, 3], [])])
        runner.step([StepEntry(cache, [4], [0])])
        assert runner.graphs.captures == 1
        gone = [weakref.ref(runner), weakref.ref(runner.graphs), weakref.ref(runner.storage)]
        del runner, cache
        assert [r() for r in gone] == [None, None, None]
    finally:
        gc.enable()


ODD = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 72, "num_hidden_layers": 2, "num_attention_heads": 3, "num_key_value_heads": 3, "head_dim": 24,
    "intermediate_size": 100, "vocab_size": 131, "rope_theta": 5000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True, "max_position_embeddings": 200,
}


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_decoding_against_contexts_that_are_split_and_merged(tmp_path, dtype):
    """Requests of 40, 300 and 700 tokens decode together: a device with idle compute units
    gives the long ones to several work items of 128 keys whose partial results are merged, the
    short one needs no merge, and the graph of the step pads both tables.  Eagerly and through
    graphs, against the plain implementation."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    cfg = dict(helpers.TINY_B, max_position_embeddings=1024)
    d = helpers.make_model_dir(tmp_path / "long", cfg, seed=21)
    model = load_model(d, dtype=dtype)
    seqs = [helpers.token_ids(cfg["vocab_size"], n, 700 + n) for n in (40, 300, 700)]
    refs = [plain.forward_dir(d, ids).numpy() for ids in seqs]
    n_decoded = 6
    for graphs in (False, True):
        runner = Runner(model, page_size=8, num_pages=160, max_requests=4, use_graphs=graphs)
        caches = [runner.manager.open(i) for i in range(len(seqs))]
        runner.step([StepEntry(c, ids[:-n_decoded], []) for c, ids in zip(caches, seqs)])
        for t in range(n_decoded, 0, -1):
            out = runner.step([StepEntry(c, [ids[-t]], [0]) for c, ids in zip(caches, seqs)]).float().cpu().numpy()
            for i, ref in enumerate(refs):
                helpers.assert_close_to_plain(out[i:i + 1], ref[len(ref) - t:len(ref) - t + 1], dtype,
                                              f"graphs={graphs} request of {len(seqs[i])} tokens, {t} from its end")
        if graphs and runner.graphs.enabled:
            assert runner.graphs.replays >= n_decoded - 2
    if dtype == "bfloat16":  # the step that was tested is one that splits
        from types import SimpleNamespace
        host = SimpleNamespace(n_seqs=3, q_lens=[1, 1, 1], past_lens=[len(ids) - 1 for ids in seqs])
        assert model.planners[0].split_keys(host, True) == 128


def test_a_growing_batch_keeps_its_graph_while_its_items_grow_longer(tmp_path, monkeypatch):
    """Three requests decode 260 tokens each through graphs on a device that the planner takes to
    have six compute units, so that the rules for the length of attention items (halving, the
    lengths between the powers of two, the shortening that fills the last round of workgroups) all
    come into play at these small sizes: the items change their length many times, the graph of the
    batch changes only when the tables or the waves of an item double, and every 20th token's logits
    are those of the plain implementation."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine import graphs
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    monkeypatch.setattr(graphs, "CAPTURE_AFTER", 1)
    cfg = dict(helpers.TINY_B, max_position_embeddings=2048)
    d = helpers.make_model_dir(tmp_path / "grow", cfg, seed=23)
    model = load_model(d, dtype="bfloat16")
    planner = model.planners[0]
    planner.compute_units = 6
    n_decoded = 260
    seqs = [helpers.token_ids(cfg["vocab_size"], n + n_decoded, 900 + n) for n in (200, 520, 1100)]
    refs = [plain.forward_dir(d, ids).numpy() for ids in seqs]
    runner = Runner(model, page_size=16, num_pages=176, max_requests=4)
    assert runner.graphs.enabled
    caches = [runner.manager.open(i) for i in range(len(seqs))]
    runner.step([StepEntry(c, ids[:-n_decoded], []) for c, ids in zip(caches, seqs)])
    lengths = set()
    from types import SimpleNamespace
    for t in range(n_decoded, 0, -1):
        host = SimpleNamespace(n_seqs=3, q_lens=[1, 1, 1], past_lens=[len(ids) - t for ids in seqs])
        lengths.add(planner.split_keys(host, True))
        out = runner.step([StepEntry(c, [ids[-t]], [0]) for c, ids in zip(caches, seqs)])
        if t % 20 == 1:
            got = out.float().cpu().numpy()
            for i, ref in enumerate(refs):
                helpers.assert_close_to_plain(got[i:i + 1], ref[len(ref) - t:len(ref) - t + 1], "bfloat16",
                                              f"request of {len(seqs[i])} tokens, {t} from its end")
    print(f"item lengths {sorted(lengths)}, {runner.graphs.captures} graphs, {runner.graphs.replays} replays")
    assert len(lengths) >= 3, f"the items were {sorted(lengths)} keys long"
    assert runner.graphs.captures <= 4 and runner.graphs.replays >= n_decoded - 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [3, 8])
def test_sizes_the_fast_kernels_do_not_take_still_give_right_results(tmp_path, dtype, page_size):
    """A head size that is no multiple of 16, an inner size that is no multiple of 8, a vocabulary
    and a width that are no powers of two, a page size that is no multiple of 4: the matrix-core
    kernels do not take these and the engine must fall back to kernels that do, in bfloat16 too."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    d = helpers.make_model_dir(tmp_path / "odd", ODD, seed=5)
    ids = [helpers.token_ids(131, n, 600 + n) for n in (150, 41)]
    ref = [plain.forward_dir(d, x).numpy() for x in ids]
    runner = Runner(load_model(d, dtype=dtype), page_size=page_size, num_pages=96, max_requests=2)
    a, b = runner.manager.open("a"), runner.manager.open("b")
    got = {0: [], 1: []}
    plan = [[(0, 100), (1, 2)], [(0, 1), (1, 30)], [(0, 1), (1, 1)], [(0, 48), (1, 8)]]
    fed = [0, 0]
    for step in plan:
        entries = [StepEntry((a, b)[i], ids[i][fed[i]:fed[i] + n], list(range(n))) for i, n in step]
        out = runner.step(entries).cpu()
        at = 0
        for i, n in step:
            got[i].append(out[at:at + n]); at += n; fed[i] += n
    for i in (0, 1):
        helpers.assert_close_to_plain(torch.cat(got[i]).numpy(), ref[i], dtype, f"odd sizes {dtype} page {page_size} request {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_thousands_of_tokens_in_portions_of_2048(tmp_path, dtype):
    """4,600 tokens of the second tiny configuration (its position limit raised) fed in portions
    of 2,048, 2,048 and 504 tokens, then 40 tokens decoded one by one: long portions behind
    thousands of cached keys through the attention kernel that shares keys in LDS, a block table
    of 290 pages, decode items that are split and merged."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    cfg = dict(helpers.TINY_B, max_position_embeddings=8192)
    d = helpers.make_model_dir(tmp_path / "long", cfg, seed=31)
    ids = helpers.token_ids(cfg["vocab_size"], 4640, 4640)
    ref = plain.forward_dir(d, ids).numpy()
    runner = Runner(load_model(d, dtype=dtype), page_size=16, num_pages=300, max_requests=2)
    rc = runner.manager.open("long")
    fed = 0
    for n in (2048, 2048, 504):
        want = sorted(set(range(0, n, 97)) | {n - 2, n - 1})
        out = runner.step([StepEntry(rc, ids[fed:fed + n], want)]).float().cpu().numpy()
        helpers.assert_close_to_plain(out, ref[[fed + w for w in want]], dtype, f"{dtype} portion at {fed}")
        fed += n
    rows = [runner.step([StepEntry(rc, ids[t:t + 1], [0])]).float().cpu().numpy() for t in range(fed, len(ids))]
    helpers.assert_close_to_plain(np.concatenate(rows), ref[fed:], dtype, f"{dtype} decoding behind 4,600 tokens")
    runner.manager.close(rc)
    runner.manager.check_invariants()


@pytest.mark.parametrize("run_ahead", [True, False])
def test_batched_requests_that_meet_their_end_tokens_at_different_steps(llms, model_dirs, run_ahead):
    """Five requests decode together, one step ahead of the host; each has an end-of-sequence
    token of its own that the plain greedy continuation meets at another step (one never meets
    it).  A request that ends has already been run one token too far by the step in flight: that
    token is dropped, its pages go back, the others go on.  Outputs equal the plain continuation
    cut at the end token, with and without running ahead; the manager's invariants hold after
    every step."""
    from from_scratch_inference_engine_amd import Engine, SamplingParams, SeqStatus

    model = llms[("B", "float32")].model
    prompts = [helpers.token_ids(509, n, 500 + n) for n in (4, 9, 17, 30, 6)]
    free = [plain_greedy(model_dirs["B"], p, 14) for p in prompts]
    eos = [free[0][2], free[1][5], free[2][9], -1, free[4][12]]
    want = [f[:f.index(e) + 1] if e in f else f for f, e in zip(free, eos)]
    assert len({len(w) for w in want}) >= 4  # they do end at different steps
    engine = Engine(model, block_size=8, num_blocks=40, max_batch=8)
    engine.run_ahead = run_ahead
    ids = [engine.add_request(p, SamplingParams(temperature=0.0), max_tokens=14, eos_id=e) for p, e in zip(prompts, eos)]
    steps = 0
    while engine.has_work():
        engine.step()
        engine.runner.manager.check_invariants()
        steps += 1
        assert steps < 100
    assert [engine.output(i) for i in ids] == want
    assert all(engine.status(i) == SeqStatus.Finished for i in ids)
    assert engine.free_blocks() == 40 and engine.runner.manager.free_slots == 8


def test_more_requests_than_a_step_has_tokens_for(llms, model_dirs):
    """A token budget smaller than the number of requests asked to run at once: the engine never
    runs more requests than a step has tokens for, so nobody who decodes is left out of a step;
    the others wait their turn.  Outputs are the plain continuations."""
    from from_scratch_inference_engine_amd import Engine, SamplingParams

    model = llms[("A", "float32")].model
    engine = Engine(model, block_size=4, num_blocks=64, max_batch=6, max_tokens_per_step=4)
    assert engine.scheduler.max_batch == 4
    prompts = [helpers.token_ids(256, n, 600 + n) for n in (3, 5, 2, 7, 4, 6)]
    got = engine.generate_batch(prompts, SamplingParams(temperature=0.0), max_tokens=8)
    assert got == [plain_greedy(model_dirs["A"], p, 8) for p in prompts]
    assert engine.free_blocks() == 64


def _model_with_one_loud_key(tmp_path, special, layer=0):
    """The second tiny configuration with one layer (the first, or a later one, whose input still
    carries the token's embedding beside the small sums of the layers before) arranged so that every query gives
    nearly all of its attention to the keys of one token, wherever it stands: dimension 15 of the
    key (the slowest-turning rotary pair: the rotation leaves it alone over thousands of positions)
    reads how much the normed input looks like that token's, and every query head carries a
    large constant there.  Near-uniform attention, which random weights give, would hide a key
    that is missed or taken from the wrong page; here the logits move by a whole unit."""
    cfg = dict(helpers.TINY_B, max_position_embeddings=2048)
    t = {k: v.float() for k, v in helpers.random_tensors(cfg, 1).items()}
    p = f"model.layers.{layer}."
    n = plain.rms_norm(t["model.embed_tokens.weight"][special][None], t[p + "input_layernorm.weight"], 1e-5)[0]
    t[p + "self_attn.k_proj.weight"][15] = 8.0 * n / (n @ n)
    t[p + "self_attn.k_proj.bias"][15] = 0.0
    for h in range(6):
        t[p + "self_attn.q_proj.weight"][h * 32 + 15] = 0.0
        t[p + "self_attn.q_proj.bias"][h * 32 + 15] = 40.0
    return helpers.make_model_dir(tmp_path / "loud", cfg, 1, tensors={k: v.to(torch.bfloat16).contiguous() for k, v in t.items()})


@pytest.mark.parametrize("dtype, layer", [("bfloat16", 0), ("float32", 0), ("bfloat16", 2)])
def test_the_model_finds_one_far_key_through_its_own_tables(tmp_path, dtype, layer):
    """Three requests whose loud token stands at position 2, at the last slot of a page and 1,200
    tokens back: prefilled in portions beside each other's decoded tokens, then decoded together
    (eagerly and through graphs).  What the step function's tables and the attention plan hand
    to the kernels decides the logits here.  With the last layer made loud instead of the first, a
    key taken from another layer's plane of the pool shows in bfloat16 too."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    special = 100
    d = _model_with_one_loud_key(tmp_path, special, layer)
    seqs = []
    for n, where, seed in ((700, 2, 1), (420, 335, 2), (1500, 287, 3)):
        ids = [t if t != special else special + 1 for t in helpers.token_ids(509, n, 880 + seed)]
        ids[where] = special
        seqs.append(ids)
    cfg, w = plain.read_config(d), plain.read_weights(d)
    refs = [plain.forward(cfg, w, ids).numpy() for ids in seqs]
    # the construction does what it says: without the loud token the later logits are far away
    quiet = list(seqs[1])
    quiet[335] = special + 1
    assert np.abs(plain.forward(cfg, w, quiet).numpy()[400:] - refs[1][400:]).max() > 0.5
    model = load_model(d, dtype=dtype)
    for graphs in (False, True):
        runner = Runner(model, page_size=16, num_pages=200, max_requests=4, use_graphs=graphs)
        caches = [runner.manager.open(i) for i in range(3)]
        fed = [0, 0, 0]
        got = [[], [], []]
        # portions of different sizes beside each other; request 1 is already decoding while 2 is in its prompt
        plan = [[(0, 300), (1, 410)], [(0, 392), (1, 1), (2, 700)], [(1, 1), (2, 2)], [(0, 1), (1, 1), (2, 791)]]
        plan += [[(0, 1), (1, 1), (2, 1)]] * 7
        for step in plan:
            entries = [StepEntry(caches[i], seqs[i][fed[i]:fed[i] + n], [n - 1]) for i, n in step]
            out = runner.step(entries).float().cpu().numpy()
            for row, (i, n) in enumerate(step):
                fed[i] += n
                got[i].append((fed[i] - 1, out[row]))
        for i in range(3):
            assert fed[i] == len(seqs[i])
            pos = [p for p, _ in got[i]]
            helpers.assert_close_to_plain(np.stack([r for _, r in got[i]]), refs[i][pos], dtype,
                                          f"{dtype} graphs={graphs} request {i}")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_what_an_earlier_request_left_in_its_pages_does_not_reach_the_next(model_dirs, dtype):
    """Every page of the pools is filled with NaN, as a request whose activations overflowed would
    leave them (all but the null page, which nothing ever writes).  A request that takes such a
    page finds it zeroed, and keys it has no page for are read from the null page: a probability
    of zero times what lies there is zero.  Portions, decoded tokens and a batch padded to a
    graph's size (whose filler rows live in the spare page) all give the plain model's logits."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    model = load_model(model_dirs["A"], dtype=dtype)
    seqs = [helpers.token_ids(256, n, 1300 + n) for n in (37, 22, 9)]
    refs = [plain.forward_dir(model_dirs["A"], ids).numpy() for ids in seqs]
    for graphs in (False, True):
        runner = Runner(model, page_size=4, num_pages=24, max_requests=4, use_graphs=graphs)
        k, v, _ = runner.storage.group_stores[0]
        k[:, 1:] = float("nan")
        v[:, 1:] = float("nan")
        caches = [runner.manager.open(i) for i in range(3)]
        fed = [0, 0, 0]
        plan = [[(0, 30), (1, 2)], [(0, 1), (1, 13), (2, 3)], [(0, 1), (1, 1), (2, 1)], [(0, 1), (1, 1), (2, 1)],
                [(0, 4), (1, 5), (2, 4)]]
        for step in plan:
            entries = [StepEntry(caches[i], seqs[i][fed[i]:fed[i] + n], list(range(n))) for i, n in step]
            out = runner.step(entries).float().cpu().numpy()
            row = 0
            for i, n in step:
                helpers.assert_close_to_plain(out[row:row + n], refs[i][fed[i]:fed[i] + n], dtype,
                                              f"{dtype} graphs={graphs} request {i} at {fed[i]}")
                row += n
                fed[i] += n
        assert fed == [len(s_) for s_ in seqs]
        assert not torch.isnan(k[:, 0]).any() and (k[:, 0] == 0).all() and (v[:, 0] == 0).all()  # the null page stays empty


def test_nan_in_the_pools_and_the_attention_that_finishes_qkv_itself(tmp_path):
    """The same for the kernel of steps of one token a request, which writes the new key and value
    into the pools while other waves of its workgroup read the 16 bytes around that place (masked
    by a probability of zero): what lies in the slots at and after a request's length must be
    finite, and it is, because a page is zeroed by the step that takes it, whatever an earlier
    request left there.  A configuration that this kernel takes (head size 32, pages of 8, a hidden
    size of 1,024 that the sliced product takes); requests decode across the edges of their pages, in pages
    that another request, closed meanwhile, had filled."""
    from from_scratch_inference_engine_amd import load_model, ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    cfg = dict(WIDE, head_dim=32, num_attention_heads=8, max_position_embeddings=256)  # hidden 1,024: two slices of K
    d = helpers.make_model_dir(tmp_path / "m", cfg, seed=77)
    model = load_model(d, dtype="bfloat16")
    seqs = [helpers.token_ids(331, n, 1500 + n) for n in (29, 14, 21)]
    refs = [plain.forward_dir(d, ids).numpy() for ids in seqs]
    calls = []
    real = ops.attention_mfma_qkv
    ops.attention_mfma_qkv = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        for graphs in (False, True):
            runner = Runner(model, page_size=8, num_pages=9, max_requests=3, use_graphs=graphs)
            k, v, _ = runner.storage.group_stores[0]
            k[:, 1:] = float("nan")
            v[:, 1:] = float("nan")
            calls.clear()
            a, b = runner.manager.open("a"), runner.manager.open("b")
            fed = {"a": 0, "b": 0, "c": 0}
            which = {"a": 0, "b": 1, "c": 2}
            caches = {"a": a, "b": b}

            def step(items):
                entries = [StepEntry(caches[r], seqs[which[r]][fed[r]:fed[r] + n], list(range(n))) for r, n in items]
                out = runner.step(entries).float().cpu().numpy()
                row = 0
                for r, n in items:
                    helpers.assert_close_to_plain(out[row:row + n], refs[which[r]][fed[r]:fed[r] + n], "bfloat16",
                                                  f"graphs={graphs} request {r} at {fed[r]}")
                    row += n
                    fed[r] += n

            step([("a", 5), ("b", 6)])
            for _ in range(8):                     # both decode over the edge of their first page (8)
                step([("a", 1), ("b", 1)])
            runner.manager.close(caches.pop("b"))  # b's two pages, filled with its keys, go back ...
            k[:, 1:][torch.isfinite(k[:, 1:])] = float("nan")  # ... and whatever they held is made worse
            v[:, 1:][torch.isfinite(v[:, 1:])] = float("nan")
            caches["c"] = runner.manager.open("c")
            # a's keys are gone with that (they were finite): it starts again in pages of its own
            runner.manager.close(caches.pop("a"))
            caches["a"] = runner.manager.open("a")
            fed["a"] = 0
            step([("a", 9), ("c", 3)])
            for _ in range(18):                    # c runs into b's old pages, one token a step, a beside it
                step([("a", 1), ("c", 1)])
            assert fed == {"a": 27, "b": 14, "c": 21}
            assert len(calls) >= (26 * 2 if not graphs else 2), "the kernel that finishes q/k/v ran"
            assert (k[:, 0] == 0).all() and (v[:, 0] == 0).all()
    finally:
        ops.attention_mfma_qkv = real


def test_steps_filled_up_to_the_timed_row_counts_of_256_and_more(tmp_path):
    """With the library's kernels chosen by timing, a step of 448 tokens (two requests' portions) is
    filled up to 512 rows with the tokens of a request that does not exist, and a step of 300
    stays as it is (512 would add more than a fifth); the real requests' logits are the plain
    model's either way, and so is what they decode next."""
    from from_scratch_inference_engine_amd import load_model, ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry, padded_tokens
    from from_scratch_inference_engine_amd.engine.model import Runner

    assert padded_tokens(448) == 512 and padded_tokens(300) == 300 and padded_tokens(1000) == 1024
    cfg = dict(helpers.TINY_B, max_position_embeddings=1024)
    d = helpers.make_model_dir(tmp_path / "m", cfg, seed=41)
    seqs = [helpers.token_ids(509, n, 1400 + n) for n in (301, 149, 302)]
    refs = [plain.forward_dir(d, ids).numpy() for ids in seqs]
    rows_seen = []
    real_mm = ops.library_mm
    ops.enable_library_tuning(max_ms_per_candidate=5, iterations=2)
    try:
        runner = Runner(load_model(d, dtype="bfloat16"), page_size=16, num_pages=80, max_requests=4,
                        fill_rows=padded_tokens)
        import from_scratch_inference_engine_amd.parts.linear as linear_module
        saved = linear_module.library_mm
        linear_module.library_mm = lambda x, w, **k: (rows_seen.append(x.shape[0]), saved(x, w, **k))[1]
        try:
            caches = [runner.manager.open(i) for i in range(3)]
            # 300 + 148 = 448 tokens: filled up to 512
            out = runner.step([StepEntry(caches[0], seqs[0][:300], [299]), StepEntry(caches[1], seqs[1][:148], [0, 147])]).float().cpu().numpy()
            helpers.assert_close_to_plain(out[:1], refs[0][299:300], "bfloat16", "filled-up step, request 0")
            helpers.assert_close_to_plain(out[1:], refs[1][[0, 147]], "bfloat16", "filled-up step, request 1")
            assert set(rows_seen) == {512}, set(rows_seen)
            rows_seen.clear()
            # 300 tokens alone: as they are
            out = runner.step([StepEntry(caches[2], seqs[2][:300], [299])]).float().cpu().numpy()
            helpers.assert_close_to_plain(out, refs[2][299:300], "bfloat16", "a step of 300 rows")
            assert set(rows_seen) == {300}, set(rows_seen)
            # the next tokens of all three, decoded together
            out = runner.step([StepEntry(c, [s_[len(s_) - 1 - (len(s_) == 302)]], [0]) for c, s_ in zip(caches, seqs)]).float().cpu().numpy()
            for i, (s_, at) in enumerate(zip(seqs, (300, 148, 300))):
                helpers.assert_close_to_plain(out[i:i + 1], refs[i][at:at + 1], "bfloat16", f"decoding after it, request {i}")
        finally:
            linear_module.library_mm = saved
    finally:
        ops.disable_library_tuning()
    assert ops.library_mm is real_mm
