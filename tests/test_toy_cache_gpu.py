"""Parts with caches and arrangements that the engine does not have, defined here and run
without a change to the engine's files:

* a mixer whose per-token cache is one float32 vector (no keys, no values), through a cache need
  of its own that allocates its pool and hands out its view;
* a mixer with a running state that takes the step from device tables alone, so that its decode
  steps are replayed from graphs: its state must advance once per step, also in the step that
  captures the graph;
* a block that normalises the mixer's output before it is added (a sandwich), through the norm's
  entry for plain tensors.
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
    from from_scratch_inference_engine_amd.cache import StateNeed
    from from_scratch_inference_engine_amd.cache.needs import CacheNeed
    from from_scratch_inference_engine_amd.config.base import ModelConfig, required_int
    from from_scratch_inference_engine_amd.models import LayerCall, ModelSpec, bind, register_architecture
    from from_scratch_inference_engine_amd.parts import (Block, LMHead, Mixer, ParamDecl, TokenEmbedding, make_part,
                                                         register_part)
    from from_scratch_inference_engine_amd.weights import TensorSpec

    @dataclass(frozen=True)
    class VectorNeed(CacheNeed):
        """One float32 vector of ``dim`` values per token and layer, whatever the compute dtype."""

        dim: int
        window = None
        per_token = True

        def allocate(self, n_caches, units, page_size, device, dtype):
            return torch.zeros((n_caches, units, page_size, self.dim), dtype=torch.float32, device=device)

        def view(self, store, plane, ctx, group, writes):
            return SimpleNamespace(pool=store[plane], block_tables=ctx.block_tables[group], slots=ctx.slots[group],
                                   page_size=store.shape[2], writes=writes)

        def bytes_per_token(self, dtype):
            return 4 * self.dim

        def store_bytes(self, store):
            return store.numel() * 4

    @register_part("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """u_t = x_t W_in^T is kept per token (float32, in pages); y_t = mean(u_0..u_t) W_out^T."""

        def __init__(self, hidden_size: int, dim: int):
            self.hidden_size, self.dim = hidden_size, dim
            self.w_in = self.w_out = None

        def param_decls(self):
            return {"w_in": ParamDecl((self.dim, self.hidden_size)), "w_out": ParamDecl((self.hidden_size, self.dim))}

        def cache_need(self):
            return VectorNeed(self.dim)

        def forward(self, x, ctx, cache):
            u = x.float() @ self.w_in.float().t()
            flat = cache.pool.view(-1, self.dim)
            flat[cache.slots.long()] = u  # every token's entry at its slot
            out = torch.empty((x.shape[0], self.hidden_size), dtype=x.dtype, device=x.device)
            host, ps = ctx.host, cache.page_size
            for s in range(ctx.n_seqs):
                total = host.past_lens[s] + host.q_lens[s]
                pos = torch.arange(total, device=x.device)
                entries = flat[cache.block_tables[s].long()[pos // ps] * ps + pos % ps]  # gathered through the block table
                means = entries.cumsum(0)[host.past_lens[s]:] / (pos[host.past_lens[s]:] + 1).unsqueeze(1)
                out[host.q_starts[s]:host.q_starts[s + 1]] = (means @ self.w_out.float().t()).to(x.dtype)
            return out

    @register_part("mixer", "toy_decay_on_device")
    class DecayOnDevice(Mixer):
        """s_t = decay * s_{t-1} + x_t, y_t = s_t W^T, the state in the request's slot.  Everything
        that changes from step to step comes from the device tables (the host gives shapes only)."""

        graph_safe = True

        def __init__(self, hidden_size: int, decay: float):
            self.hidden_size, self.decay = hidden_size, decay
            self.weight = None

        def param_decls(self):
            return {"weight": ParamDecl((self.hidden_size, self.hidden_size))}

        def cache_need(self):
            return StateNeed((self.hidden_size,), "float32")

        def forward(self, x, ctx, cache):
            out = torch.empty_like(x)
            q_lens = ctx.host.q_lens
            slots = ctx.seq_slots.long()
            starts = ctx.q_starts.long()
            for j in range(max(q_lens)):
                if all(n > j for n in q_lens):
                    rows, at = starts[:-1] + j, slots
                else:
                    keep = torch.tensor([s for s, n in enumerate(q_lens) if n > j], device=x.device)
                    rows, at = starts[:-1][keep] + j, slots[keep]
                state = cache.state[at] * self.decay + x[rows].float()
                cache.state[at] = state
                out[rows] = (state @ self.weight.float().t()).to(x.dtype)
            return out

    @register_part("block", "toy_sandwich")
    class Sandwich(Block):
        """x += post(mixer(norm1(x))); x += ffn(norm2(x)): the mixer's output is normalised before
        it joins the stream."""

        def __init__(self, mixer_norm, mixer, post_norm, ffn_norm, ffn):
            self.mixer_norm, self.mixer, self.post_norm, self.ffn_norm, self.ffn = mixer_norm, mixer, post_norm, ffn_norm, ffn

        def sub_parts(self):
            return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "post_norm": self.post_norm,
                    "ffn_norm": self.ffn_norm, "ffn": self.ffn}

        def forward(self, hidden, ctx, cache):
            x = self.mixer_norm(hidden, ctx.compute_dtype)
            hidden.delta = self.post_norm.plain(self.mixer.forward(x, ctx, cache))
            x = self.ffn_norm(hidden, ctx.compute_dtype)
            hidden.delta = self.ffn.forward(x, ctx)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        hidden_size: int = 0
        vocab_size: int = 0
        num_layers: int = 0
        mixer: str = ""
        dim: int = 0
        decay: float = 0.5
        inter: int = 0
        eps: float = 1e-6
        longest: int = 0

        @property
        def max_positions(self):
            return self.longest  # this architecture keeps its limit under a key of its own

        @classmethod
        def from_dict(cls, raw):
            return cls(architecture=raw["architectures"][0], hidden_size=required_int(raw, "hidden_size"),
                       vocab_size=required_int(raw, "vocab_size"), num_layers=required_int(raw, "num_layers"),
                       mixer=raw["mixer"], dim=int(raw.get("dim", 0)), decay=float(raw.get("decay", 0.5)),
                       inter=required_int(raw, "inter"), eps=float(raw["eps"]), longest=int(raw.get("longest", 0)))

    def build(cfg: ToyConfig) -> ModelSpec:
        h, bindings, layers = cfg.hidden_size, [], []
        emb = TokenEmbedding(cfg.vocab_size, h)
        bind(bindings, emb, "weight", [TensorSpec("emb", (cfg.vocab_size, h))])
        norm_of = lambda name: make_part("norm", "rms_norm", hidden_size=h, eps=cfg.eps)
        for l in range(cfg.num_layers):
            if cfg.mixer == "mean":
                mixer = make_part("mixer", "toy_running_mean", hidden_size=h, dim=cfg.dim)
                bind(bindings, mixer, "w_in", [TensorSpec(f"l{l}.in", (cfg.dim, h))])
                bind(bindings, mixer, "w_out", [TensorSpec(f"l{l}.out", (h, cfg.dim))])
            else:
                mixer = make_part("mixer", "toy_decay_on_device", hidden_size=h, decay=cfg.decay)
                bind(bindings, mixer, "weight", [TensorSpec(f"l{l}.mix", (h, h))])
            ffn = make_part("feed_forward", "swiglu", hidden_size=h, intermediate_size=cfg.inter)
            n1, n2 = norm_of("n1"), norm_of("n2")
            if cfg.mixer == "mean":
                post = norm_of("post")
                layers.append(make_part("block", "toy_sandwich", mixer_norm=n1, mixer=mixer, post_norm=post, ffn_norm=n2, ffn=ffn))
                bind(bindings, post, "weight", [TensorSpec(f"l{l}.post", (h,), "norm")])
            else:
                layers.append(make_part("block", "pre_norm", mixer_norm=n1, mixer=mixer, ffn_norm=n2, ffn=ffn))
            bind(bindings, n1, "weight", [TensorSpec(f"l{l}.n1", (h,), "norm")])
            bind(bindings, n2, "weight", [TensorSpec(f"l{l}.n2", (h,), "norm")])
            bind(bindings, ffn, "gate_up_weight", [TensorSpec(f"l{l}.gate", (cfg.inter, h)), TensorSpec(f"l{l}.up", (cfg.inter, h))])
            bind(bindings, ffn, "down_weight", [TensorSpec(f"l{l}.down", (h, cfg.inter))])
        norm = norm_of("norm")
        bind(bindings, norm, "weight", [TensorSpec("norm", (h,), "norm")])
        head = LMHead(h, cfg.vocab_size)
        bind(bindings, head, "weight", [TensorSpec("emb", (cfg.vocab_size, h))])
        return ModelSpec(config=cfg, embedding=emb, layers=layers, schedule=[LayerCall(l) for l in range(cfg.num_layers)],
                         final_norm=norm, lm_head=head, bindings=bindings)

    register_architecture("ToyCacheLM", ToyConfig, build)
    return ToyConfig


def plain_toy(raw, w, ids):
    x = w["emb"][torch.tensor(ids)]
    for l in range(raw["num_layers"]):
        n1 = plain.rms_norm(x, w[f"l{l}.n1"], raw["eps"])
        if raw["mixer"] == "mean":
            u = n1 @ w[f"l{l}.in"].t()
            means = u.cumsum(0) / torch.arange(1, len(ids) + 1).unsqueeze(1)
            x = x + plain.rms_norm(means @ w[f"l{l}.out"].t(), w[f"l{l}.post"], raw["eps"])
        else:
            s, mixed = torch.zeros(raw["hidden_size"]), []
            for t in range(len(ids)):
                s = raw["decay"] * s + n1[t]
                mixed.append(s @ w[f"l{l}.mix"].t())
            x = x + torch.stack(mixed)
        n2 = plain.rms_norm(x, w[f"l{l}.n2"], raw["eps"])
        x = x + plain.linear(plain.silu_mul(plain.linear(n2, w[f"l{l}.gate"]), plain.linear(n2, w[f"l{l}.up"])), w[f"l{l}.down"])
    return plain.linear(plain.rms_norm(x, w["norm"], raw["eps"]), w["emb"])


def _make(tmp_path, raw, seed):
    from from_scratch_inference_engine_amd import load_config, load_model
    from from_scratch_inference_engine_amd.weights import SafetensorsFile, write_random_model

    d = tmp_path / raw["mixer"]
    d.mkdir()
    (d / "config.json").write_text(json.dumps(raw))
    cfg = load_config(d)
    object.__setattr__(cfg, "to_dict", lambda: raw)
    write_random_model(cfg, seed, d, torch.float32)
    f = SafetensorsFile(d / "model.safetensors")
    return load_model(d, dtype="float32"), {n: f.get(n).clone() for n in f.names()}


def test_a_per_token_cache_of_one_vector_and_a_sandwich_norm(tmp_path):
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    define_toys()
    raw = {"architectures": ["ToyCacheLM"], "hidden_size": 40, "vocab_size": 83, "num_layers": 2, "mixer": "mean",
           "dim": 12, "inter": 56, "eps": 1e-5, "longest": 64}
    model, w = _make(tmp_path, raw, 6)
    layout = model.cache_layout
    assert len(layout.paged_groups) == 1 and type(layout.paged_groups[0]).__name__ == "VectorNeed"
    assert layout.group_caches == [[0, 1]] and model.cache_bytes_per_token() == 2 * 4 * 12
    runner = Runner(model, page_size=4, num_pages=14, max_requests=3)
    store = runner.storage.group_stores[0]
    assert store.shape == (2, 16, 4, 12)  # null page, 14 pages, spare page and store.dtype == torch.float32 and runner.storage.bytes() == store.numel() * 4
    assert runner.max_position == 64  # read through the typed configuration, whatever the key is called
    seqs = {"a": helpers.token_ids(83, 30, 1), "b": helpers.token_ids(83, 11, 2), "c": helpers.token_ids(83, 17, 3)}
    ref = {k: plain_toy(raw, w, ids) for k, ids in seqs.items()}
    caches, fed, got = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    # "c" starts when "b" has ended and takes its pages
    plan = [[("a", 6), ("b", 11)], [("a", 1)], [("a", 2), ("c", 3)], [("c", 1), ("a", 1)], [("c", 13), ("a", 20)]]
    for step in plan:
        entries = []
        for k, n in step:
            if k not in caches:
                if k == "c":
                    runner.manager.close(caches.pop("b"))
                caches[k] = runner.manager.open(k)
            entries.append(StepEntry(caches[k], seqs[k][fed[k]:fed[k] + n], list(range(n))))
            fed[k] += n
        out = runner.step(entries).cpu()
        row = 0
        for e in entries:
            got[e.cache.request_id].append(out[row:row + len(e.tokens)])
            row += len(e.tokens)
        runner.manager.check_invariants()
    for k in seqs:
        assert fed[k] == len(seqs[k])
        assert (torch.cat(got[k]) - ref[k]).abs().max() <= 1e-4, k
    assert runner.manager.allocators[0].pages_issued_again()
    with pytest.raises(ValueError, match="limit of 64"):
        runner.step([StepEntry(runner.manager.open("long"), [1] * 65, [])])


def test_a_state_on_the_device_advances_once_a_step_through_graphs(tmp_path):
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    define_toys()
    raw = {"architectures": ["ToyCacheLM"], "hidden_size": 48, "vocab_size": 97, "num_layers": 2, "mixer": "decay",
           "decay": 0.8, "inter": 72, "eps": 1e-5}
    model, w = _make(tmp_path, raw, 4)
    seqs = [helpers.token_ids(97, 19 + 4 * i, 40 + i) for i in range(3)]
    ref = [plain_toy(raw, w, ids) for ids in seqs]
    for graphs in (True, False):
        runner = Runner(model, page_size=4, num_pages=4, max_requests=4, use_graphs=graphs)
        assert runner.graphs is None or runner.graphs.enabled  # every part reads device tables: graphs are on
        caches = [runner.manager.open(i) for i in range(3)]
        n_pre = [len(ids) - 9 for ids in seqs]
        out = runner.step([StepEntry(c, ids[:n], [n - 1]) for c, ids, n in zip(caches, seqs, n_pre)]).cpu()
        for i in range(3):
            assert (out[i] - ref[i][n_pre[i] - 1]).abs().max() <= 1e-4
        for t in range(9):  # the first of these captures the graph (three requests in a graph of four rows)
            out = runner.step([StepEntry(c, [ids[n + t]], [0]) for c, ids, n in zip(caches, seqs, n_pre)]).cpu()
            torch.cuda.synchronize()
            _ = (torch.randn(64, 64, device="cuda") @ torch.randn(64, 64, device="cuda")).sum().item()
            for i in range(3):
                assert (out[i] - ref[i][n_pre[i] + t]).abs().max() <= 1e-4, f"graphs={graphs} request {i} token {t}"
        if graphs:
            assert runner.graphs.captures == 1 and runner.graphs.replays == 8
        # a request that starts in a slot that was used finds its state zero: one token, alone
        runner.manager.close(caches[1])
        late = runner.manager.open("late")
        assert late.slot == caches[1].slot
        out = runner.step([StepEntry(late, seqs[2][:1], [0])]).cpu()
        assert (out[0] - ref[2][0]).abs().max() <= 1e-4


def test_norm_of_plain_tensors_whole_rows_and_heads():
    from from_scratch_inference_engine_amd import ops

    for dtype in (torch.float32, torch.bfloat16):
        g = torch.Generator().manual_seed(3)
        x = torch.randn(7, 6 * 40, generator=g).to(dtype)
        w_row, w_head = torch.randn(240, generator=g) + 1.0, torch.randn(40, generator=g) + 1.0
        tol = 1e-5 if dtype == torch.float32 else 2.0 ** -7 * 4
        out = ops.rmsnorm_plain(x.cuda(), w_row.cuda(), 1e-5).float().cpu()
        assert (out - plain.rms_norm(x.float(), w_row, 1e-5)).abs().max() <= tol
        # per head: runs of 40, in place, on the first four heads of rows that are 240 apart
        dev = x.clone().cuda()
        ops.rmsnorm_plain(dev[:, :160], w_head.cuda(), 1e-6, out=dev[:, :160])
        want = plain.rms_norm(x.float()[:, :160].reshape(7 * 4, 40), w_head, 1e-6).reshape(7, 160)
        assert (dev.float().cpu()[:, :160] - want).abs().max() <= tol
        assert torch.equal(dev.cpu()[:, 160:], x[:, 160:])
    with pytest.raises(ops.KernelError, match="whole runs"):
        ops.rmsnorm_plain(torch.zeros(2, 10).cuda(), torch.ones(4).cuda(), 1e-6)
