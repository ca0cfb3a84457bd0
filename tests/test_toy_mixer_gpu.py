"""A mixer with state of its own, defined here, is registered, built and stepped without a change
to the engine's files: a new architecture name, a configuration class, a mixer that keeps a
fixed-size state per request in the cache manager's slots."""

import json

import numpy as np
import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu


def define_toy():
    from dataclasses import dataclass

    from from_scratch_inference_engine_amd.cache import StateNeed
    from from_scratch_inference_engine_amd.config.base import ModelConfig, required_int
    from from_scratch_inference_engine_amd.models import LayerCall, ModelSpec, bind, register_architecture
    from from_scratch_inference_engine_amd.parts import (LMHead, Mixer, ParamDecl, TokenEmbedding, make_part,
                                                         register_part)
    from from_scratch_inference_engine_amd.weights import TensorSpec

    @register_part("mixer", "toy_decay_state")
    class DecayMixer(Mixer):
        """y_t = s_t W^T with s_t = decay * s_{t-1} + x_t: a running, decaying sum over the
        request's tokens.  The state s (one vector per request) lives in the cache's state slots,
        so that a portion continues where the last one stopped."""

        def __init__(self, hidden_size: int, decay: float):
            self.hidden_size, self.decay = hidden_size, decay
            self.weight = None

        def param_decls(self):
            return {"weight": ParamDecl((self.hidden_size, self.hidden_size))}

        def cache_need(self):
            return StateNeed((self.hidden_size,), "float32")

        def forward(self, x, ctx, cache):
            out = torch.empty_like(x)
            for s in range(ctx.n_seqs):  # the toy walks the host's view of the batch, token by token
                lo, hi, slot = ctx.host.q_starts[s], ctx.host.q_starts[s + 1], ctx.host.seq_slots[s]
                state = cache.state[slot]
                for t in range(lo, hi):
                    state.mul_(self.decay).add_(x[t].float())
                    out[t] = (state @ self.weight.float().t()).to(x.dtype)
            return out

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        hidden_size: int = 0
        vocab_size: int = 0
        num_layers: int = 0
        decay: float = 0.5
        inter: int = 0
        eps: float = 1e-6

        @classmethod
        def from_dict(cls, raw):
            return cls(architecture=raw["architectures"][0], hidden_size=required_int(raw, "hidden_size"),
                       vocab_size=required_int(raw, "vocab_size"), num_layers=required_int(raw, "num_layers"),
                       decay=float(raw["decay"]), inter=required_int(raw, "inter"), eps=float(raw["eps"]))

    def build(cfg: ToyConfig) -> ModelSpec:
        bindings = []
        emb = TokenEmbedding(cfg.vocab_size, cfg.hidden_size)
        bind(bindings, emb, "weight", [TensorSpec("emb", (cfg.vocab_size, cfg.hidden_size))])
        layers = []
        for l in range(cfg.num_layers):
            mixer = make_part("mixer", "toy_decay_state", hidden_size=cfg.hidden_size, decay=cfg.decay)
            ffn = make_part("feed_forward", "swiglu", hidden_size=cfg.hidden_size, intermediate_size=cfg.inter)
            n1 = make_part("norm", "rms_norm", hidden_size=cfg.hidden_size, eps=cfg.eps)
            n2 = make_part("norm", "rms_norm", hidden_size=cfg.hidden_size, eps=cfg.eps)
            layers.append(make_part("block", "pre_norm", mixer_norm=n1, mixer=mixer, ffn_norm=n2, ffn=ffn))
            bind(bindings, mixer, "weight", [TensorSpec(f"l{l}.mix", (cfg.hidden_size, cfg.hidden_size))])
            bind(bindings, n1, "weight", [TensorSpec(f"l{l}.n1", (cfg.hidden_size,), "norm")])
            bind(bindings, n2, "weight", [TensorSpec(f"l{l}.n2", (cfg.hidden_size,), "norm")])
            bind(bindings, ffn, "gate_up_weight", [TensorSpec(f"l{l}.gate", (cfg.inter, cfg.hidden_size)),
                                                   TensorSpec(f"l{l}.up", (cfg.inter, cfg.hidden_size))])
            bind(bindings, ffn, "down_weight", [TensorSpec(f"l{l}.down", (cfg.hidden_size, cfg.inter))])
        norm = make_part("norm", "rms_norm", hidden_size=cfg.hidden_size, eps=cfg.eps)
        bind(bindings, norm, "weight", [TensorSpec("norm", (cfg.hidden_size,), "norm")])
        head = LMHead(cfg.hidden_size, cfg.vocab_size)
        bind(bindings, head, "weight", [TensorSpec("emb", (cfg.vocab_size, cfg.hidden_size))])
        return ModelSpec(config=cfg, embedding=emb, layers=layers, schedule=[LayerCall(l) for l in range(cfg.num_layers)],
                         final_norm=norm, lm_head=head, bindings=bindings)

    register_architecture("ToyDecayLM", ToyConfig, build)
    return ToyConfig


def plain_toy(raw, w, ids):
    import plain_qwen2 as plain

    x = w["emb"][torch.tensor(ids)]
    for l in range(raw["num_layers"]):
        n1 = plain.rms_norm(x, w[f"l{l}.n1"], raw["eps"])
        s = torch.zeros(raw["hidden_size"])
        mixed = []
        for t in range(len(ids)):
            s = raw["decay"] * s + n1[t]
            mixed.append(s @ w[f"l{l}.mix"].t())
        x = x + torch.stack(mixed)
        n2 = plain.rms_norm(x, w[f"l{l}.n2"], raw["eps"])
        x = x + plain.linear(plain.silu_mul(plain.linear(n2, w[f"l{l}.gate"]), plain.linear(n2, w[f"l{l}.up"])), w[f"l{l}.down"])
    return plain.linear(plain.rms_norm(x, w["norm"], raw["eps"]), w["emb"])


def test_toy_state_mixer_is_registered_built_and_stepped(tmp_path):
    from from_scratch_inference_engine_amd import load_config, load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner
    from from_scratch_inference_engine_amd.weights import write_random_model, SafetensorsFile

    ToyConfig = define_toy()
    raw = {"architectures": ["ToyDecayLM"], "hidden_size": 48, "vocab_size": 97, "num_layers": 2, "decay": 0.8,
           "inter": 72, "eps": 1e-5}
    (tmp_path / "m").mkdir()
    (tmp_path / "m" / "config.json").write_text(json.dumps(raw))
    cfg = load_config(tmp_path / "m")
    assert isinstance(cfg, ToyConfig)
    object.__setattr__(cfg, "to_dict", lambda: raw)
    write_random_model(cfg, 4, tmp_path / "m", torch.float32)  # the random-weights mode works for it too
    f = SafetensorsFile(tmp_path / "m" / "model.safetensors")
    w = {n: f.get(n).clone() for n in f.names()}
    model = load_model(tmp_path / "m", dtype="float32")
    assert model.cache_layout.paged_groups == [] and len(model.cache_layout.state_caches) == 2
    runner = Runner(model, page_size=4, num_pages=4, max_requests=3)
    assert runner.graphs.enabled is False  # the toy reads the host's view: no graph replay for this model
    seqs = {"a": helpers.token_ids(97, 23, 1), "b": helpers.token_ids(97, 9, 2), "c": helpers.token_ids(97, 14, 3)}
    ref = {k: plain_toy(raw, w, ids) for k, ids in seqs.items()}
    got = {k: [] for k in seqs}
    caches = {k: runner.manager.open(k) for k in ("a", "b")}
    fed = {k: 0 for k in seqs}
    plan = [[("a", 5), ("b", 9)], [("a", 1)], [("a", 2), ("c", 3)], [("c", 11), ("a", 15)]]
    for step in plan:
        entries = []
        for k, n in step:
            if k not in caches:  # "c" takes the slot that "b" gave back: its state must start from zero
                runner.manager.close(caches.pop("b"))
                caches[k] = runner.manager.open(k)
                assert caches[k].slot == 1
            entries.append(StepEntry(caches[k], seqs[k][fed[k]:fed[k] + n], list(range(n))))
            fed[k] += n
        out = runner.step(entries).cpu()
        row = 0
        for e in entries:
            got[e.cache.request_id].append(out[row:row + len(e.tokens)])
            row += len(e.tokens)
    for k in seqs:
        assert fed[k] == len(seqs[k])
        assert (torch.cat(got[k]) - ref[k]).abs().max() <= 1e-4, k
