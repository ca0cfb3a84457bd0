"""Pins the plain implementation by what fixes it beside the reference's text: the vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake (wrong sign or pairing, a norm in the wrong place) fails."""

import math

import pytest
import torch

import plain_qwen2 as plain


# ---- vectors from the reference's tests (tests/cpp/test_nn.cpp, test_tensor.cpp, test_sampler.cpp)
def test_linear_vectors():
    y = plain.linear(torch.tensor([[1.0, 2.0]]), torch.ones(2, 2), torch.tensor([10.0, 20.0]))
    assert y.tolist() == [[13.0, 23.0]]  # test_nn.cpp:8-17
    y = plain.linear(torch.tensor([[1.0, 2.0, 3.0]]), torch.tensor([[1.0, 0, 0], [0, 1.0, 0]]))
    assert y.tolist() == [[1.0, 2.0]]  # test_nn.cpp:19-25
    x = torch.tensor([[1.0, 2, 3], [4, 5, 6]])
    w_t = torch.tensor([[7.0, 8], [9, 10], [11, 12]])  # [K, N]; the weight is its transpose
    assert plain.linear(x, w_t.t().contiguous()).flatten().tolist() == [58.0, 64.0, 139.0, 154.0]  # test_tensor.cpp:32-43


def test_rms_norm_vector_and_placement_of_eps_and_weight():
    y = plain.rms_norm(torch.tensor([[3.0, 4.0]]), torch.ones(2), 0.0)
    s = 1.0 / math.sqrt(12.5)  # test_nn.cpp:27-34
    assert y.flatten().tolist() == pytest.approx([3 * s, 4 * s], abs=1e-6)
    # eps is inside the square root and added to the mean, not to the sum or outside
    y = plain.rms_norm(torch.tensor([[3.0, 4.0]]), torch.ones(2), 1.0)
    assert y.flatten().tolist() == pytest.approx([3 / math.sqrt(13.5), 4 / math.sqrt(13.5)], abs=1e-6)
    # the weight multiplies (plain w, not 1 + w), after the normalisation
    y = plain.rms_norm(torch.tensor([[3.0, 4.0]]), torch.tensor([2.0, 0.0]), 0.0)
    assert y.flatten().tolist() == pytest.approx([6 * s, 0.0], abs=1e-6)
    # scale invariance at eps = 0 and unit RMS at w = 1
    x = torch.randn(5, 37, generator=torch.Generator().manual_seed(0))
    a, b = plain.rms_norm(x, torch.ones(37), 0.0), plain.rms_norm(7.5 * x, torch.ones(37), 0.0)
    assert torch.allclose(a, b, atol=1e-6)
    assert torch.allclose((a * a).mean(-1), torch.ones(5), atol=1e-5)
    assert torch.equal(plain.rms_norm(torch.zeros(1, 4), torch.ones(4), 1e-6), torch.zeros(1, 4))


def test_silu_mul_vector():
    y = plain.silu_mul(torch.tensor([0.0, 1.0]), torch.tensor([5.0, 2.0]))  # test_nn.cpp:36-42
    assert y.tolist() == pytest.approx([0.0, 2.0 / (1.0 + math.exp(-1.0))], abs=1e-6)
    big = plain.silu_mul(torch.tensor([30.0]), torch.tensor([3.0]))
    assert big.item() == pytest.approx(90.0, rel=1e-6)
    assert torch.allclose(plain.silu_mul(torch.tensor([-1.3, 0.7]), torch.tensor([1.0, 1.0])),
                          torch.nn.functional.silu(torch.tensor([-1.3, 0.7])), atol=1e-7)


def test_embedding_vectors():
    w = torch.tensor([[0.0, 1], [2, 3], [4, 5]])
    assert plain.embedding(w, [2, 0]).flatten().tolist() == [4.0, 5.0, 0.0, 1.0]  # test_nn.cpp:44-51
    with pytest.raises(IndexError):
        plain.embedding(torch.zeros(2, 2), [5])  # test_nn.cpp:53-56


def test_rope_vector_sign_and_pairing():
    y = plain.rope(torch.tensor([[1.0, 0.0]]), 1, 2, 10000.0, [1])  # test_nn.cpp:58-64
    assert y.flatten().tolist() == pytest.approx([math.cos(1.0), math.sin(1.0)], abs=1e-6)
    # pairing is (i, i + half), not (2i, 2i + 1): a unit vector at index 0 of a 4-wide head
    # spreads into indices 0 and 2 only
    y = plain.rope(torch.tensor([[1.0, 0.0, 0.0, 0.0]]), 1, 4, 10000.0, [3]).flatten()
    assert y[1].item() == 0.0 and y[3].item() == 0.0
    assert y[0].item() == pytest.approx(math.cos(3.0), abs=1e-6)
    assert y[2].item() == pytest.approx(math.sin(3.0), abs=1e-6)
    # second pair turns with frequency theta^(-2/4)
    y = plain.rope(torch.tensor([[0.0, 1.0, 0.0, 0.0]]), 1, 4, 10000.0, [3]).flatten()
    f = 10000.0 ** (-0.5)
    assert y.tolist() == pytest.approx([0.0, math.cos(3 * f), 0.0, math.sin(3 * f)], abs=1e-6)


def test_rope_is_a_complex_rotation_and_keeps_relative_positions():
    g = torch.Generator().manual_seed(1)
    hd, heads = 16, 3
    x = torch.randn(6, heads * hd, generator=g)
    pos = [0, 1, 5, 17, 100, 4095]
    y = plain.rope(x, heads, hd, 1e6, pos)
    assert torch.equal(y[0], x[0])  # position 0 is the identity
    xc = torch.complex(x.double().reshape(6, heads, hd)[..., :hd // 2], x.double().reshape(6, heads, hd)[..., hd // 2:])
    inv = torch.tensor([1e6 ** (-2.0 * i / hd) for i in range(hd // 2)], dtype=torch.float64)
    ang = torch.tensor(pos, dtype=torch.float64).reshape(6, 1, 1) * inv
    yc = xc * torch.polar(torch.ones_like(ang), ang)
    want = torch.cat([yc.real, yc.imag], dim=-1).reshape(6, heads * hd).float()
    assert torch.allclose(y, want, atol=1e-6)
    # q.k after RoPE depends only on the distance between the positions
    q, k = torch.randn(1, hd, generator=g), torch.randn(1, hd, generator=g)
    def dot(pq, pk):
        return (plain.rope(q, 1, hd, 1e4, [pq]) * plain.rope(k, 1, hd, 1e4, [pk])).sum().item()
    assert dot(7, 3) == pytest.approx(dot(107, 103), abs=1e-5)
    assert dot(7, 3) != pytest.approx(dot(3, 7), abs=1e-3)  # and on its sign


def test_attention_first_row_is_value():
    q = torch.tensor([[0.3, -0.1], [0.5, 0.2]])
    k = torch.tensor([[0.1, 0.4], [-0.2, 0.3]])
    v = torch.tensor([[7.0, 8.0], [1.0, 2.0]])
    o = plain.attention(q, k, v, 1, 1, 2)  # test_nn.cpp:66-74
    assert o[0].tolist() == pytest.approx([7.0, 8.0], abs=1e-6)


def test_attention_last_row_is_library_softmax_attention():
    """The last query sees every key: softmax(q K^T / sqrt(d)) V per head, kv heads repeated."""
    g = torch.Generator().manual_seed(2)
    s, nh, nkv, hd = 9, 4, 2, 8
    q, k, v = torch.randn(s, nh * hd, generator=g), torch.randn(s, nkv * hd, generator=g), torch.randn(s, nkv * hd, generator=g)
    o = plain.attention(q, k, v, nh, nkv, hd)
    kk = k.reshape(s, nkv, hd).repeat_interleave(nh // nkv, dim=1)  # consecutive q heads share a kv head
    vv = v.reshape(s, nkv, hd).repeat_interleave(nh // nkv, dim=1)
    for h in range(nh):
        w = torch.softmax((q[-1].reshape(nh, hd)[h] @ kk[:, h].t()) / math.sqrt(hd), dim=-1)
        assert torch.allclose(o[-1].reshape(nh, hd)[h], w @ vv[:, h], atol=1e-6)
    # every row i equals the last row of the problem cut after i (causality)
    for i in (0, 3):
        oi = plain.attention(q[:i + 1], k[:i + 1], v[:i + 1], nh, nkv, hd)
        assert torch.allclose(oi[-1], o[i], atol=1e-6)
    # n_kv = n_heads is plain multi-head attention through torch's routine
    k2, v2 = torch.randn(s, nh * hd, generator=g), torch.randn(s, nh * hd, generator=g)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.reshape(s, nh, hd).transpose(0, 1), k2.reshape(s, nh, hd).transpose(0, 1),
        v2.reshape(s, nh, hd).transpose(0, 1), is_causal=True).transpose(0, 1).reshape(s, nh * hd)
    assert torch.allclose(plain.attention(q, k2, v2, nh, nh, hd), want, atol=1e-5)


def test_attention_invariants():
    g = torch.Generator().manual_seed(3)
    s, hd = 6, 4
    q, v = torch.randn(s, hd, generator=g), torch.randn(s, hd, generator=g)
    k = torch.randn(1, hd, generator=g).repeat(s, 1)  # identical keys: running mean of the values
    o = plain.attention(q, k, v, 1, 1, hd)
    want = torch.cumsum(v, 0) / torch.arange(1, s + 1).reshape(s, 1)
    assert torch.allclose(o, want, atol=1e-6)
    # query offset: rows of a later portion equal the same rows of the whole
    k = torch.randn(s, hd, generator=g)
    whole = plain.attention(q, k, v, 1, 1, hd)
    part = plain.attention(q[4:], k, v, 1, 1, hd, query_offset=4)
    assert torch.allclose(part, whole[4:], atol=1e-7)
    # a window of w positions: the query at p reads p-w+1..p
    win = plain.attention(q, k, v, 1, 1, hd, window=2)
    two = plain.attention(q[4:5], k[3:5], v[3:5], 1, 1, hd, query_offset=1)
    assert torch.allclose(win[4], two[0], atol=1e-7)


def test_model_is_causal_and_head_choice(model_dirs):
    cfg, w = plain.read_config(model_dirs["A"]), plain.read_weights(model_dirs["A"])
    assert cfg["head_dim"] == 16 and cfg["qkv_bias"] is True  # derived head_dim, qwen2 bias
    ids = [3, 9, 200, 41, 7, 7, 19]
    full = plain.forward(cfg, w, ids)
    assert full.shape == (7, 256)
    assert torch.allclose(plain.forward(cfg, w, ids[:4]), full[:4], atol=1e-6)
    # tied: the head is the embedding table; untied: lm_head.weight
    assert "lm_head.weight" not in w
    cfg_b, w_b = plain.read_config(model_dirs["B"]), plain.read_weights(model_dirs["B"])
    out = plain.forward(cfg_b, w_b, [1, 2, 3])
    w_b2 = dict(w_b)
    w_b2["lm_head.weight"] = w_b["lm_head.weight"] * 2
    assert torch.allclose(plain.forward(cfg_b, w_b2, [1, 2, 3]), out * 2, atol=1e-6)


# ---- sampler (tests/cpp/test_sampler.cpp:7-56)
def test_sampler_vectors():
    assert plain.sample(torch.tensor([0.1, 0.2, 5.0, 0.3]), 0.0, 0, 1.0, 0.3) == 2
    assert plain.argmax(torch.tensor([0.0, 1.0, 5.0, 1.0, 0.0, 5.0])) == 2  # first maximum wins
    for u in (0.0, 0.3, 0.999):
        assert plain.sample(torch.tensor([1.0, 3.0, 2.0]), 1.0, 1, 1.0, u) == 1  # top_k = 1
        assert plain.sample(torch.tensor([0.0, 10.0, 0.0, 0.0]), 1.0, 0, 0.5, u) == 1  # top_p keeps the dominant
    n = 2000
    hits = sum(plain.sample(torch.tensor([0.0, 2.0, 0.0]), 1.0, 0, 1.0, (i + 0.5) / n) == 1 for i in range(n))
    assert abs(hits / n - 0.7869) < 0.002  # softmax([0, 2, 0])[1]
    # temperature sharpens: at T = 0.1 nearly everything goes to the top token
    hits = sum(plain.sample(torch.tensor([0.0, 2.0, 0.0]), 0.1, 0, 1.0, (i + 0.5) / 200) == 1 for i in range(200))
    assert hits == 200
    # vocabulary order of the draw: small u gives the first kept token
    assert plain.sample(torch.tensor([1.0, 1.0, 1.0]), 1.0, 0, 1.0, 0.01) == 0
    assert plain.sample(torch.tensor([1.0, 1.0, 1.0]), 1.0, 0, 1.0, 0.99) == 2


# ---- the whole model's composition (src/model/model.cpp:90-149), pinned without any package's
# model code: special cases in which the model reduces to a few library routines, a second
# composition written from torch's own routines only, and an invariant of the positions
def _library_model(cfg, w, ids):
    """The decoder put together from torch's library routines alone (embedding, rms_norm, linear,
    silu, scaled_dot_product_attention, complex multiplication for the rotation), in float64 so
    that it owes nothing to the plain implementation's choices of precision."""
    import torch.nn.functional as F

    nh, nkv, hd, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    w = {k: v.double() for k, v in w.items()}
    s = len(ids)
    x = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    ang = torch.arange(s, dtype=torch.float64)[:, None] * cfg["rope_theta"] ** (
        -torch.arange(0, hd, 2, dtype=torch.float64) / hd)[None, :]
    turn = torch.polar(torch.ones_like(ang), ang)[:, None, :]  # [S, 1, hd/2]

    def rotate(t, heads):
        t = t.reshape(s, heads, hd)
        z = torch.complex(t[..., :hd // 2], t[..., hd // 2:]) * turn
        return torch.cat([z.real, z.imag], dim=-1)

    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = F.rms_norm(x, (x.shape[-1],), w[p + "input_layernorm.weight"], eps)
        q = rotate(F.linear(h, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]), nh)
        k = rotate(F.linear(h, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]), nkv)
        v = F.linear(h, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).reshape(s, nkv, hd)
        k, v = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
        a = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        x = x + F.linear(a.transpose(0, 1).reshape(s, nh * hd), w[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (x.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    x = F.rms_norm(x, (x.shape[-1],), w["model.norm.weight"], eps)
    return F.linear(x, w.get("lm_head.weight", w["model.embed_tokens.weight"]))


@pytest.mark.parametrize("name", ["A", "B"])
def test_whole_model_equals_a_composition_of_library_routines(model_dirs, name):
    import helpers

    cfg, w = plain.read_config(model_dirs[name]), plain.read_weights(model_dirs[name])
    ids = helpers.token_ids(cfg["vocab_size"], 41, 123)
    got, want = plain.forward(cfg, w, ids).double(), _library_model(cfg, w, ids)
    assert (got - want).abs().max().item() <= 1e-5
    assert torch.equal(got.argmax(-1), want.argmax(-1))


def _one_layer(seed=0, **sizes):
    """A one-layer model with larger weights than the tiny ones, so that every term is visible."""
    cfg = {"hidden_size": 24, "num_hidden_layers": 1, "num_attention_heads": 3, "num_key_value_heads": 1,
           "head_dim": 8, "intermediate_size": 20, "vocab_size": 31, "rope_theta": 100.0, "rms_norm_eps": 1e-3,
           "qkv_bias": True}
    cfg.update(sizes)
    g = torch.Generator().manual_seed(seed)
    h, nh, nkv, hd, it, v = (cfg[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                                                "intermediate_size", "vocab_size"))
    r = lambda *shape: torch.randn(*shape, generator=g) * 0.5
    p = "model.layers.0."
    w = {"model.embed_tokens.weight": r(v, h), "model.norm.weight": 1 + r(h), "lm_head.weight": r(v, h),
         p + "input_layernorm.weight": 1 + r(h), p + "post_attention_layernorm.weight": 1 + r(h),
         p + "self_attn.q_proj.weight": r(nh * hd, h), p + "self_attn.q_proj.bias": r(nh * hd),
         p + "self_attn.k_proj.weight": r(nkv * hd, h), p + "self_attn.k_proj.bias": r(nkv * hd),
         p + "self_attn.v_proj.weight": r(nkv * hd, h), p + "self_attn.v_proj.bias": r(nkv * hd),
         p + "self_attn.o_proj.weight": r(h, nh * hd), p + "mlp.gate_proj.weight": r(it, h),
         p + "mlp.up_proj.weight": r(it, h), p + "mlp.down_proj.weight": r(h, it)}
    return cfg, w


def test_model_special_cases_reduce_to_library_routines():
    import torch.nn.functional as F

    cfg, w = _one_layer()
    p, eps, ids = "model.layers.0.", cfg["rms_norm_eps"], [5, 30, 5, 11]
    x = w["model.embed_tokens.weight"][ids]
    head = lambda t: F.linear(F.rms_norm(t, (t.shape[-1],), w["model.norm.weight"], eps), w["lm_head.weight"])
    # both residual branches silenced: logits = head(norm(embedding)); no scaling of the embedding
    w0 = dict(w)
    w0[p + "self_attn.o_proj.weight"] = torch.zeros_like(w[p + "self_attn.o_proj.weight"])
    w0[p + "mlp.down_proj.weight"] = torch.zeros_like(w[p + "mlp.down_proj.weight"])
    assert torch.allclose(plain.forward(cfg, w0, ids), head(x), atol=1e-5)
    # attention silenced: x + down(silu(gate(n2(x))) * up(n2(x))); swapping gate and up must show
    w1 = dict(w)
    w1[p + "self_attn.o_proj.weight"] = w0[p + "self_attn.o_proj.weight"]
    n2 = F.rms_norm(x, (x.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
    mlp = F.linear(F.silu(F.linear(n2, w[p + "mlp.gate_proj.weight"])) * F.linear(n2, w[p + "mlp.up_proj.weight"]),
                   w[p + "mlp.down_proj.weight"])
    got = plain.forward(cfg, w1, ids)
    assert torch.allclose(got, head(x + mlp), atol=1e-5)
    swapped = dict(w1)
    swapped[p + "mlp.gate_proj.weight"], swapped[p + "mlp.up_proj.weight"] = w[p + "mlp.up_proj.weight"], w[p + "mlp.gate_proj.weight"]
    assert (plain.forward(cfg, swapped, ids) - got).abs().max() > 1e-2
    # feed-forward silenced, one token: attention over one key is its value, so the layer is
    # x + o(v(n1(x)) + b_v) repeated for every head of the group: bias on v, none on o, the first
    # norm before the projections, the residual taken from before the norm
    w2 = dict(w)
    w2[p + "mlp.down_proj.weight"] = w0[p + "mlp.down_proj.weight"]
    x1 = x[:1]
    n1 = F.rms_norm(x1, (x1.shape[-1],), w[p + "input_layernorm.weight"], eps)
    v = F.linear(n1, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"])
    a = v.reshape(1, cfg["num_key_value_heads"], cfg["head_dim"]).repeat_interleave(
        cfg["num_attention_heads"] // cfg["num_key_value_heads"], dim=1).reshape(1, -1)
    assert torch.allclose(plain.forward(cfg, w2, ids[:1]), head(x1 + F.linear(a, w[p + "self_attn.o_proj.weight"])), atol=1e-5)
    # the biases of q and k count (a model that dropped them gives other logits for two tokens)
    nob = dict(w2)
    nob[p + "self_attn.q_proj.bias"] = torch.zeros_like(w[p + "self_attn.q_proj.bias"])
    assert (plain.forward(cfg, nob, ids) - plain.forward(cfg, w2, ids)).abs().max() > 1e-4


def test_model_depends_on_distances_only_and_rotates_q_and_k_but_not_v(monkeypatch):
    """All positions shifted by a constant: the logits stay (only distances count), which a
    rotation of the values, or of q alone, would break."""
    cfg, w = _one_layer(seed=1, num_attention_heads=4, num_key_value_heads=2, hidden_size=32)
    ids = [1, 2, 3, 4, 5, 6, 7]
    base = plain.forward(cfg, w, ids)
    real = plain.rope
    monkeypatch.setattr(plain, "rope", lambda x, nh, hd, theta, pos: real(x, nh, hd, theta, [p + 1000 for p in pos]))
    assert torch.allclose(plain.forward(cfg, w, ids), base, atol=2e-5)
    # the check can fail: rotating only what has as many heads as q (q alone) changes the logits
    monkeypatch.setattr(plain, "rope", lambda x, nh, hd, theta, pos:
                        real(x, nh, hd, theta, [p + 1000 for p in pos]) if nh == 4 else real(x, nh, hd, theta, pos))
    assert (plain.forward(cfg, w, ids) - base).abs().max() > 1e-3
