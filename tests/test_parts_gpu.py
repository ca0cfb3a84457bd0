"""Each part of a layer alone, on the GPU, against the plain functions; then arrangements that
the Qwen2 model itself does not use (a window, a layer run twice, a layer that reads another
layer's cache) through toy architectures registered by the test."""

import json
import math

import numpy as np
import pytest
import torch

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, seed, dtype=torch.float32, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def tol(dtype, ref, f32=2e-5):
    return f32 * max(1.0, ref.abs().max().item()) if dtype == torch.float32 else 2.0 ** -6 * ref.abs().max().item()


class Ctx:
    """The least a norm or feed-forward needs of a step."""

    def __init__(self, dtype):
        self.compute_dtype = dtype


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    from from_scratch_inference_engine_amd.parts import HiddenState, make_part

    norm = make_part("norm", "rms_norm", hidden_size=200, eps=3e-4)
    assert norm.param_decls()["weight"].shape == (200,) and norm.param_decls()["weight"].storage == "vector"
    norm.weight = (rnd((200,), 1) + 1).cuda()
    x, d = rnd((6, 200), 2), rnd((6, 200), 3, dtype)
    hidden = HiddenState(x.clone().cuda(), d.cuda())
    out = norm(hidden, dtype).float().cpu()
    ref = plain.rms_norm(x + d.float(), norm.weight.cpu(), 3e-4)
    assert hidden.delta is None and torch.equal(hidden.residual.cpu(), x + d.float())  # the sum was folded in
    assert (out - ref).abs().max() <= tol(dtype, ref)
    hidden = HiddenState(x.clone().cuda(), d.cuda())
    rows = torch.tensor([5, 1], dtype=torch.int32).cuda()
    out = norm.rows(hidden, rows, dtype).float().cpu()
    assert (out - ref[[5, 1]]).abs().max() <= tol(dtype, ref) and hidden.delta is not None


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(dtype):
    from from_scratch_inference_engine_amd.parts import make_part

    ffn = make_part("feed_forward", "swiglu", hidden_size=96, intermediate_size=200)
    assert ffn.param_decls()["gate_up_weight"].shape == (400, 96)
    gate, up, down = rnd((200, 96), 4, dtype, 0.1), rnd((200, 96), 5, dtype, 0.1), rnd((96, 200), 6, dtype, 0.1)
    assert ffn.param_decls()["gate_up_weight"].layout == "interleave"
    ffn.gate_up_weight = torch.stack([gate, up], dim=1).reshape(400, 96).cuda()  # g0, u0, g1, u1, ...
    ffn.down_weight = down.cuda()
    for rows in (3, 40):  # the small-matrix kernel with its fused epilogue, and the library product
        x = rnd((rows, 96), 7, dtype)
        out = ffn.forward(x.cuda(), Ctx(dtype)).float().cpu()
        ref = plain.linear(plain.silu_mul(plain.linear(x.float(), gate.float()), plain.linear(x.float(), up.float())), down.float())
        assert (out - ref).abs().max() <= tol(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_parts(dtype):
    from from_scratch_inference_engine_amd.parts import LMHead, TokenEmbedding

    emb, head = TokenEmbedding(301, 72), LMHead(72, 301)
    table = rnd((301, 72), 8, dtype)
    emb.weight = table.cuda()
    head.weight = emb.weight  # tied
    ids = torch.tensor([300, 0, 7], dtype=torch.int32)
    x = emb.forward(ids.cuda())
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table.float()[ids.long()])
    h = rnd((5, 72), 9, dtype)
    logits = head.forward(h.cuda())
    assert logits.dtype == torch.float32
    ref = plain.linear(h.float(), table.float())
    assert (logits.cpu() - ref).abs().max() <= 2e-5 * ref.abs().max() + 1e-6


def mixer_harness(mixer, dtype, page_size, num_pages, n_requests=3):
    """A cache and a context maker for one mixer, from the engine's public pieces."""
    from from_scratch_inference_engine_amd.cache import CacheManager
    from from_scratch_inference_engine_amd.cache.storage import CacheLayout, CacheStorage
    from from_scratch_inference_engine_amd.engine.context import PinnedStaging, StepEntry, build_context
    from from_scratch_inference_engine_amd.parts import prepare_parts

    prepare_parts(mixer, "cuda", dtype)
    manager = CacheManager([mixer.cache_need()], page_size, num_pages, n_requests)
    storage = CacheStorage(CacheLayout([mixer.cache_need()], [[0]], {}), manager, "cuda", dtype)
    staging = PinnedStaging()

    def run(items):
        """items: list of (request cache, x [n, H]); returns the mixer's output rows."""
        entries = [StepEntry(rc, [0] * x.shape[0], []) for rc, x in items]
        for e in entries:
            manager.reserve(e.cache, len(e.tokens))
        ctx, _ = build_context(entries, manager, [mixer.planner()], staging, dtype, "cuda")
        out = mixer.forward(torch.cat([x for _, x in items]).cuda(), ctx, storage.view(0, ctx, writes=True))
        for e in entries:
            manager.commit(e.cache, len(e.tokens))
        return out.float().cpu()

    return manager, run


def plain_attention_mixer(x, wq, wk, wv, bq, bk, bv, wo, heads, kv, hd, theta, window=None, rope=True):
    q, k, v = plain.linear(x, wq, bq), plain.linear(x, wk, bk), plain.linear(x, wv, bv)
    if rope:
        pos = list(range(x.shape[0]))
        q, k = plain.rope(q, heads, hd, theta, pos), plain.rope(k, kv, hd, theta, pos)
    return plain.linear(plain.attention(q, k, v, heads, kv, hd, 0, window=window), wo)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv, hd, window, rope", [(6, 3, 32, None, True), (4, 1, 48, 21, True), (2, 2, 64, None, False)])
def test_attention_mixer_alone(dtype, heads, kv, hd, window, rope):
    """Portions, decoding and two requests side by side through the mixer and its pages; with a
    window the manager hands passed pages back while the mixer goes on."""
    from from_scratch_inference_engine_amd.parts import make_part

    hidden, theta, page = 80, 2e4, 4
    position = make_part("position", "rope", head_dim=hd, theta=theta) if rope else make_part("position", "none", head_dim=hd)
    mixer = make_part("mixer", "gqa_attention", hidden_size=hidden, n_heads=heads, n_kv_heads=kv, head_dim=hd,
                      qkv_bias=True, position=position, window=window)
    w = {n: rnd(s, i + 20, dtype, 0.15) for i, (n, s) in enumerate(
        [("q", (heads * hd, hidden)), ("k", (kv * hd, hidden)), ("v", (kv * hd, hidden)), ("o", (hidden, heads * hd))])}
    b = {n: rnd((s,), i + 30, torch.float32, 0.1) for i, (n, s) in enumerate([("q", heads * hd), ("k", kv * hd), ("v", kv * hd)])}
    mixer.qkv_weight = torch.cat([w["q"], w["k"], w["v"]]).cuda()
    mixer.qkv_bias = torch.cat([b["q"], b["k"], b["v"]]).cuda()
    mixer.o_weight = w["o"].cuda()
    n_pages = 40 if window is None else 24
    manager, run = mixer_harness(mixer, dtype, page, n_pages)
    xs = {"a": rnd((70, hidden), 40, dtype), "b": rnd((45, hidden), 41, dtype)}
    ref = {k: plain_attention_mixer(x.float(), w["q"].float(), w["k"].float(), w["v"].float(), b["q"], b["k"], b["v"],
                                    w["o"].float(), heads, kv, hd, theta, window, rope) for k, x in xs.items()}
    ca, cb = manager.open("a"), manager.open("b")
    got = {"a": [], "b": []}
    cuts_a, cuts_b = [17, 2, 30, 1, 1, 19], [1, 44]
    ia = ib = 0
    for step in range(max(len(cuts_a), len(cuts_b))):
        items = []
        if step < len(cuts_a):
            items.append((ca, xs["a"][ia:ia + cuts_a[step]])); ia += cuts_a[step]
        if step < len(cuts_b):
            items.append((cb, xs["b"][ib:ib + cuts_b[step]])); ib += cuts_b[step]
        out = run(items)
        row = 0
        for rc, x in items:
            got[rc.request_id].append(out[row:row + x.shape[0]]); row += x.shape[0]
        manager.check_invariants()
    for k in xs:
        o = torch.cat(got[k])
        assert (o - ref[k]).abs().max() <= tol(dtype, ref[k], f32=1e-5), k
    if window is not None:
        assert ca.tables[0][0] == -1 and ca.pages_held(0) <= -(-(window + 19) // page) + 1  # passed pages went back
        assert manager.free_pages() >= n_pages - ca.pages_held(0) - cb.pages_held(0)


# ------------------------------------------------------------------------------ arrangements
def toy_spec(cfg, layer_calls, window=None):
    """A Qwen2-like model from the engine's parts with a schedule of its own."""
    from from_scratch_inference_engine_amd.models import LayerCall, ModelSpec, bind
    from from_scratch_inference_engine_amd.models.qwen2 import build_qwen2

    spec = build_qwen2(cfg)
    if window is not None:
        for block in spec.layers:
            block.mixer.window = window
            block.mixer._planner = None
    spec.schedule = [LayerCall(*c) for c in layer_calls]
    return spec


def plain_scheduled(cfg_dict, w, ids, layer_calls, window=None):
    """The plain model with layers run in the given order; a call (l, j) reads the keys and
    values that call j computed instead of making its own."""
    nh, nkv = cfg_dict["num_attention_heads"], cfg_dict.get("num_key_value_heads", cfg_dict["num_attention_heads"])
    hd = cfg_dict.get("head_dim", cfg_dict["hidden_size"] // nh)
    theta, eps = cfg_dict["rope_theta"], cfg_dict["rms_norm_eps"]
    pos = list(range(len(ids)))
    x = plain.embedding(w["model.embed_tokens.weight"], ids)
    kept = []
    for call in layer_calls:
        l, src = call[0], (call[1] if len(call) > 1 else None)
        p = f"model.layers.{l}."
        n1 = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
        q = plain.rope(plain.linear(n1, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]), nh, hd, theta, pos)
        if src is None:
            k = plain.rope(plain.linear(n1, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]), nkv, hd, theta, pos)
            v = plain.linear(n1, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"])
        else:
            k, v = kept[src]
        kept.append((k, v))
        a = plain.attention(q, k, v, nh, nkv, hd, 0, window=window)
        x = x + plain.linear(a, w[p + "self_attn.o_proj.weight"])
        x = x + plain.mlp_block(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p)
    x = plain.rms_norm(x, w["model.norm.weight"], eps)
    return plain.linear(x, w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("calls, window", [
    ([(0,), (1,), (0,), (2,)], None),        # layer 0 runs twice: shared weights, a cache for each call
    ([(0,), (1, 0), (2,)], None),            # the second call reads the first call's keys and values
    ([(0,), (1,), (2,)], 19),                # every layer with a window of 19 positions
])
def test_schedules_and_windows(model_dirs, tmp_path, dtype, calls, window):
    from from_scratch_inference_engine_amd.config import Qwen2Config
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Model, Runner
    from from_scratch_inference_engine_amd.models import register_architecture

    name = f"ToyScheduled{abs(hash((tuple(calls), window))) % 10 ** 8}"
    register_architecture(name, Qwen2Config, lambda cfg: toy_spec(cfg, calls, window))
    raw = dict(helpers.TINY_B, architectures=[name])
    d = helpers.make_model_dir(tmp_path / "toy", raw, seed=1)  # same seed as B: same tensors
    model = Model.from_pretrained(d, dtype=dtype)
    n_caches = sum(1 for c in calls if len(c) == 1)
    assert sum(len(ids) for ids in model.cache_layout.group_caches) == n_caches
    runner = Runner(model, page_size=4, num_pages=40 if window is None else 16, max_requests=2)
    ids = helpers.token_ids(509, 90, 77)
    ref = plain_scheduled(raw, plain.read_weights(d), ids, calls, window).numpy()
    rc = runner.manager.open("x")
    outs, i = [], 0
    for n in [13, 2, 40, 1, 1, 1, 7, 25]:
        outs.append(runner.step([StepEntry(rc, ids[i:i + n], list(range(n)))]).cpu())
        i += n
    assert i == 90
    helpers.assert_close_to_plain(torch.cat(outs).numpy(), ref, dtype, f"{calls} window {window}")
    if window is not None:
        assert rc.pages_held(0) <= -(-(window + 25) // 4) + 1 < 90 // 4
    runner.manager.close(rc)
    runner.manager.check_invariants()
