"""Two more arrangements that the engine's own model does not have, defined here and run without a
change to the engine's files:

* attention whose q and k heads are normalised between the projection and the rotation (the
  engine's attention takes the norms as parts), with the engine's rotation, with no position
  encoding, and beside a layer without such norms: every way the mixer can order bias, norms,
  rotation and cache write, in both precisions, decode steps replayed from graphs;
* a mixer that keeps one cache entry per block of four tokens in pages of two entries, beside an
  attention layer whose pages hold four tokens: two groups of pages with different geometries in
  one model, counted and addressed by the cache manager and the step's tables.
"""

import json
from dataclasses import dataclass
from types import SimpleNamespace

import pytest
import torch

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu


def define_toys():
    from from_scratch_inference_engine_amd.cache.needs import CacheNeed
    from from_scratch_inference_engine_amd.config.base import ModelConfig, required_int
    from from_scratch_inference_engine_amd.models import LayerCall, ModelSpec, bind, register_architecture
    from from_scratch_inference_engine_amd.parts import LMHead, Mixer, ParamDecl, TokenEmbedding, make_part, register_part
    from from_scratch_inference_engine_amd.weights import TensorSpec

    @dataclass(frozen=True)
    class BlockNeed(CacheNeed):
        """One float32 vector of ``dim`` values per block of ``tokens_per_entry`` tokens, in pages
        of ``page_entries`` entries, whatever page size the cache was made with."""

        dim: int
        tokens_per_entry: int = 4
        page_entries: int = 2
        window = None
        per_token = True

        def allocate(self, n_caches, units, page_size, device, dtype):
            assert page_size == self.page_entries
            return torch.zeros((n_caches, units, page_size, self.dim), dtype=torch.float32, device=device)

        def view(self, store, plane, ctx, group, writes):
            return SimpleNamespace(pool=store[plane], block_tables=ctx.block_tables[group], slots=ctx.slots[group])

        def clear_fresh(self, store, pages):
            store[:, pages[pages >= 0].long()] = 0.0  # a page that a request takes starts as zeros

        def bytes_per_token(self, dtype):
            return 4 * self.dim // self.tokens_per_entry

        def store_bytes(self, store):
            return store.numel() * 4

    @register_part("mixer", "toy_block_sums")
    class BlockSums(Mixer):
        """u_t = x_t W_in^T; the cache keeps the sum of u over every block of four positions;
        y_t = (u_0 + ... + u_t) W_out^T, read as the sum of the request's entries before the step
        plus the step's own tokens."""

        def __init__(self, hidden_size: int, dim: int):
            self.hidden_size, self.dim = hidden_size, dim
            self.w_in = self.w_out = None

        def param_decls(self):
            return {"w_in": ParamDecl((self.dim, self.hidden_size)), "w_out": ParamDecl((self.hidden_size, self.dim))}

        def cache_need(self):
            return BlockNeed(self.dim)

        def forward(self, x, ctx, cache):
            u = x.float() @ self.w_in.float().t()
            flat = cache.pool.view(-1, self.dim)
            per_page, per_entry = cache.pool.shape[1], 4
            out = torch.empty((x.shape[0], self.hidden_size), dtype=x.dtype, device=x.device)
            host = ctx.host
            for s in range(ctx.n_seqs):
                rows = slice(host.q_starts[s], host.q_starts[s + 1])
                before = torch.zeros(self.dim, device=x.device)
                if host.past_lens[s]:
                    entry = torch.arange((host.past_lens[s] - 1) // per_entry + 1, device=x.device)
                    before = flat[cache.block_tables[s].long()[entry // per_page] * per_page + entry % per_page].sum(0)
                out[rows] = ((before + u[rows].cumsum(0)) @ self.w_out.float().t()).to(x.dtype)
            flat.index_add_(0, cache.slots.long(), u)  # every token into the entry of its block
            return out

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        hidden_size: int = 0
        vocab_size: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        inter: int = 0
        theta: float = 1e4
        eps: float = 1e-6
        layers: tuple = ()

        @classmethod
        def from_dict(cls, raw):
            ints = {k: required_int(raw, k) for k in ("hidden_size", "vocab_size", "heads", "kv_heads", "head_dim", "inter")}
            return cls(architecture=raw["architectures"][0], theta=float(raw["theta"]), eps=float(raw["eps"]),
                       layers=tuple(raw["layers"]), **ints)

    def build(cfg: ToyConfig) -> ModelSpec:
        """``layers``: per layer 'norms+rope', 'norms+none', 'rope', 'none' (attention with or without
        head norms and rotation) or 'blocks' (the mixer above)."""
        h, hd = cfg.hidden_size, cfg.head_dim
        q_dim, kv_dim = cfg.heads * hd, cfg.kv_heads * hd
        bindings = []
        emb = TokenEmbedding(cfg.vocab_size, h)
        bind(bindings, emb, "weight", [TensorSpec("emb", (cfg.vocab_size, h))])
        layers = []
        for l, kind in enumerate(cfg.layers):
            if kind == "blocks":
                mixer = make_part("mixer", "toy_block_sums", hidden_size=h, dim=24)
                bind(bindings, mixer, "w_in", [TensorSpec(f"l{l}.in", (24, h))])
                bind(bindings, mixer, "w_out", [TensorSpec(f"l{l}.out", (h, 24))])
            else:
                pos = (make_part("position", "rope", head_dim=hd, theta=cfg.theta) if kind.endswith("rope")
                       else make_part("position", "none", head_dim=hd))
                qn = kn = None
                if kind.startswith("norms"):
                    qn = make_part("norm", "rms_norm", hidden_size=hd, eps=cfg.eps)
                    kn = make_part("norm", "rms_norm", hidden_size=hd, eps=cfg.eps)
                    bind(bindings, qn, "weight", [TensorSpec(f"l{l}.qn", (hd,), "norm")])
                    bind(bindings, kn, "weight", [TensorSpec(f"l{l}.kn", (hd,), "norm")])
                mixer = make_part("mixer", "gqa_attention", hidden_size=h, n_heads=cfg.heads, n_kv_heads=cfg.kv_heads,
                                  head_dim=hd, qkv_bias=True, position=pos, window=None, q_norm=qn, k_norm=kn)
                bind(bindings, mixer, "qkv_weight", [TensorSpec(f"l{l}.q", (q_dim, h)), TensorSpec(f"l{l}.k", (kv_dim, h)),
                                                     TensorSpec(f"l{l}.v", (kv_dim, h))])
                bind(bindings, mixer, "qkv_bias", [TensorSpec(f"l{l}.qb", (q_dim,), "bias"),
                                                   TensorSpec(f"l{l}.kb", (kv_dim,), "bias"),
                                                   TensorSpec(f"l{l}.vb", (kv_dim,), "bias")])
                bind(bindings, mixer, "o_weight", [TensorSpec(f"l{l}.o", (h, q_dim))])
            ffn = make_part("feed_forward", "swiglu", hidden_size=h, intermediate_size=cfg.inter)
            n1 = make_part("norm", "rms_norm", hidden_size=h, eps=cfg.eps)
            n2 = make_part("norm", "rms_norm", hidden_size=h, eps=cfg.eps)
            layers.append(make_part("block", "pre_norm", mixer_norm=n1, mixer=mixer, ffn_norm=n2, ffn=ffn))
            bind(bindings, n1, "weight", [TensorSpec(f"l{l}.n1", (h,), "norm")])
            bind(bindings, n2, "weight", [TensorSpec(f"l{l}.n2", (h,), "norm")])
            bind(bindings, ffn, "gate_up_weight", [TensorSpec(f"l{l}.gate", (cfg.inter, h)), TensorSpec(f"l{l}.up", (cfg.inter, h))])
            bind(bindings, ffn, "down_weight", [TensorSpec(f"l{l}.down", (h, cfg.inter))])
        norm = make_part("norm", "rms_norm", hidden_size=h, eps=cfg.eps)
        bind(bindings, norm, "weight", [TensorSpec("norm", (h,), "norm")])
        head = LMHead(h, cfg.vocab_size)
        bind(bindings, head, "weight", [TensorSpec("head", (cfg.vocab_size, h))])
        return ModelSpec(config=cfg, embedding=emb, layers=layers, schedule=[LayerCall(l) for l in range(len(cfg.layers))],
                         final_norm=norm, lm_head=head, bindings=bindings)

    register_architecture("ToyHeadsLM", ToyConfig, build)
    return ToyConfig


def plain_toy(raw, w, ids):
    """The same model, whole sequence, no cache, from the plain functions."""
    hd, nh, nkv, eps = raw["head_dim"], raw["heads"], raw["kv_heads"], raw["eps"]
    t = len(ids)
    x = w["emb"][torch.tensor(ids)]
    for l, kind in enumerate(raw["layers"]):
        n1 = plain.rms_norm(x, w[f"l{l}.n1"], eps)
        if kind == "blocks":
            y = (n1 @ w[f"l{l}.in"].t()).cumsum(0) @ w[f"l{l}.out"].t()
        else:
            q = plain.linear(n1, w[f"l{l}.q"], w[f"l{l}.qb"])
            k = plain.linear(n1, w[f"l{l}.k"], w[f"l{l}.kb"])
            v = plain.linear(n1, w[f"l{l}.v"], w[f"l{l}.vb"])
            if kind.startswith("norms"):  # every head by itself, after the bias, before the rotation
                q = plain.rms_norm(q.reshape(t * nh, hd), w[f"l{l}.qn"], eps).reshape(t, nh * hd)
                k = plain.rms_norm(k.reshape(t * nkv, hd), w[f"l{l}.kn"], eps).reshape(t, nkv * hd)
            if kind.endswith("rope"):
                q = plain.rope(q, nh, hd, raw["theta"], range(t))
                k = plain.rope(k, nkv, hd, raw["theta"], range(t))
            y = plain.linear(plain.attention(q, k, v, nh, nkv, hd), w[f"l{l}.o"])
        x = x + y
        n2 = plain.rms_norm(x, w[f"l{l}.n2"], eps)
        x = x + plain.linear(plain.silu_mul(plain.linear(n2, w[f"l{l}.gate"]), plain.linear(n2, w[f"l{l}.up"])), w[f"l{l}.down"])
    return plain.linear(plain.rms_norm(x, w["norm"], eps), w["head"])


def _model_dir(tmp_path, raw, seed):
    from from_scratch_inference_engine_amd import load_config
    from from_scratch_inference_engine_amd.weights import SafetensorsFile, write_random_model, write_safetensors

    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(raw))
    cfg = load_config(d)
    object.__setattr__(cfg, "to_dict", lambda: raw)
    write_random_model(cfg, seed, d, torch.float32)
    f = SafetensorsFile(d / "model.safetensors")
    # values that bfloat16 holds exactly, so that both precisions and the plain side read the same
    # numbers; head norms with weights away from one, so that a norm left out or misplaced shows
    w = {n: f.get(n).clone().to(torch.bfloat16).float() for n in f.names()}
    for n in w:
        if n.endswith(".qn") or n.endswith(".kn"):
            w[n] = (w[n] * torch.linspace(0.5, 2.0, w[n].numel())).to(torch.bfloat16).float()
    write_safetensors(d / "model.safetensors", w)
    return d, w


def _run_plan(runner, seqs, plan, closes=None):
    from from_scratch_inference_engine_amd.engine.context import StepEntry

    got = {k: [] for k in seqs}
    caches, fed = {}, {k: 0 for k in seqs}
    for step in plan:
        entries = []
        for k, n in step:
            if k not in caches:
                if closes and k in closes:
                    runner.manager.close(caches.pop(closes[k]))  # the newcomer takes over that request's pages
                caches[k] = runner.manager.open(k)
            entries.append(StepEntry(caches[k], seqs[k][fed[k]:fed[k] + n], list(range(n))))
            fed[k] += n
        out = runner.step(entries).float().cpu()
        row = 0
        for e in entries:
            got[e.cache.request_id].append(out[row:row + len(e.tokens)])
            row += len(e.tokens)
        runner.manager.check_invariants()
    assert all(fed[k] == len(seqs[k]) for k in seqs)
    return {k: torch.cat(v) for k, v in got.items()}, caches


PLAN = [[("a", 13), ("b", 2)], [("a", 1), ("b", 7)], [("a", 2), ("c", 5)], [("c", 1), ("a", 1)], [("c", 11), ("a", 14)]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_with_norms_of_its_heads(tmp_path, dtype):
    """Layers: head norms then the rotation; head norms and no position encoding; the rotation
    alone (the mixer's fused kernels); neither.  Portions beside decoded tokens, then eight steps
    of one token a request, which a model whose parts are all graph-safe replays from graphs."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    define_toys()
    raw = {"architectures": ["ToyHeadsLM"], "hidden_size": 96, "vocab_size": 131, "heads": 6, "kv_heads": 2,
           "head_dim": 16, "inter": 80, "theta": 700.0, "eps": 1e-5, "layers": ["norms+rope", "none", "norms+none", "rope"]}
    d, w = _model_dir(tmp_path, raw, 17)
    model = load_model(d, dtype=dtype)
    mixers = [b.mixer for b in model.spec.layers]
    assert set(mixers[0].sub_parts()) == {"position", "q_norm", "k_norm"} and set(mixers[3].sub_parts()) == {"position"}
    assert mixers[0].q_norm in model.spec.all_parts() and mixers[0].q_norm not in model.spec.stream_norms()
    runner = Runner(model, page_size=4, num_pages=24, max_requests=3)
    assert runner.graphs.enabled
    seqs = {"a": helpers.token_ids(131, 39, 21), "b": helpers.token_ids(131, 9, 22), "c": helpers.token_ids(131, 25, 23)}
    ref = {k: plain_toy(raw, w, ids) for k, ids in seqs.items()}
    short = {k: v[:len(v) - 8] if k != "b" else v for k, v in seqs.items()}
    got, caches = _run_plan(runner, short, PLAN, closes={"c": "b"})
    tail = {k: [] for k in ("a", "c")}
    for i in range(8):  # the last eight tokens of a and c, one token a request a step
        out = runner.step([StepEntry(caches[k], [seqs[k][len(seqs[k]) - 8 + i]], [0]) for k in ("a", "c")]).float().cpu()
        for j, k in enumerate(("a", "c")):
            tail[k].append(out[j:j + 1])
    assert runner.graphs.replays >= 6
    for k in seqs:
        logits = torch.cat([got[k]] + tail.get(k, []))
        helpers.assert_close_to_plain(logits.numpy(), ref[k].numpy(), dtype, f"{dtype} {k}")
    # the norms matter: a model that skipped them would be far off (so the comparison above saw them)
    off = plain_toy(dict(raw, layers=["rope", "none", "none", "rope"]), w, seqs["a"])
    assert (off - ref["a"]).abs().max() > 50 * helpers.F32_ATOL


def test_a_cache_with_one_entry_per_block_of_tokens_beside_attention(tmp_path):
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    define_toys()
    raw = {"architectures": ["ToyHeadsLM"], "hidden_size": 48, "vocab_size": 89, "heads": 4, "kv_heads": 2,
           "head_dim": 16, "inter": 40, "theta": 500.0, "eps": 1e-5, "layers": ["rope", "blocks", "blocks"]}
    d, w = _model_dir(tmp_path, raw, 9)
    model = load_model(d, dtype="float32")
    assert len(model.cache_layout.paged_groups) == 2 and model.cache_layout.group_caches == [[0], [1, 2]]
    runner = Runner(model, page_size=4, num_pages=13, max_requests=3)
    m = runner.manager
    assert [m.tokens_per_page(g) for g in range(2)] == [4, 8] and m.smallest_page_tokens == 4
    assert runner.graphs.enabled is False  # the toy reads the step's shapes on the host
    seqs = {"a": helpers.token_ids(89, 31, 31), "b": helpers.token_ids(89, 9, 32), "c": helpers.token_ids(89, 17, 33)}
    ref = {k: plain_toy(raw, w, ids) for k, ids in seqs.items()}
    got, caches = _run_plan(runner, seqs, PLAN, closes={"c": "b"})
    for k in seqs:
        assert (got[k] - ref[k]).abs().max() <= 1e-4, k
    # pages by each group's own geometry: 31 positions are 8 pages of four and 4 pages of eight
    assert [len(t) for t in caches["a"].tables] == [8, 4] and [len(t) for t in caches["c"].tables] == [5, 3]
    again = [len(a.pages_issued_again()) for a in m.allocators]
    assert all(n > 0 for n in again), f"c ran in pages that b gave back, in both groups: {again}"
    for rc in list(caches.values()):
        m.close(rc)
    assert [a.num_free for a in m.allocators] == [13, 13]
