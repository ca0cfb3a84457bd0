"""Shared by the tests: the tiny configurations, model folders, traces and their replay."""

from __future__ import annotations

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent

# Two tiny configurations that differ in every size and option: head counts and groups (2 vs 6,
# i.e. MQA), head_dim (16 derived vs 32 stated), sizes that are no power of two (176, 320, 509,
# 192), layers, vocabulary, theta, eps, tied vs untied head, max positions.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 176, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 128, "hidden_act": "silu",
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 192, "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 320, "vocab_size": 509, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 256,
    "use_sliding_window": False, "eos_token_id": 7,
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1)}


def expected_tensor_shapes(cfg: dict) -> dict:
    """Checkpoint tensors of a Qwen2 config, written out by hand (not from the engine's spec)."""
    h, nh = cfg["hidden_size"], cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    hd = cfg.get("head_dim", h // nh)
    inter, v = cfg["intermediate_size"], cfg["vocab_size"]
    shapes = {"model.embed_tokens.weight": (v, h), "model.norm.weight": (h,)}
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (v, h)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        shapes.update({
            p + "input_layernorm.weight": (h,), p + "post_attention_layernorm.weight": (h,),
            p + "self_attn.q_proj.weight": (nh * hd, h), p + "self_attn.q_proj.bias": (nh * hd,),
            p + "self_attn.k_proj.weight": (nkv * hd, h), p + "self_attn.k_proj.bias": (nkv * hd,),
            p + "self_attn.v_proj.weight": (nkv * hd, h), p + "self_attn.v_proj.bias": (nkv * hd,),
            p + "self_attn.o_proj.weight": (h, nh * hd),
            p + "mlp.gate_proj.weight": (inter, h), p + "mlp.up_proj.weight": (inter, h),
            p + "mlp.down_proj.weight": (h, inter),
        })
    return shapes


def random_tensors(cfg: dict, seed: int, dtype=torch.bfloat16, std: float = 0.02) -> dict:
    """Weights N(0, std), norm weights 1 + N(0, std), biases N(0, std); the test's own
    generator, written with the safetensors package, so the engine's loader meets a file it did
    not write."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(expected_tensor_shapes(cfg).items()):
        t = torch.randn(shape, generator=g) * std
        if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
            t = t + 1.0
        out[name] = t.to(dtype)
    return out


def make_model_dir(path, cfg: dict, seed: int, dtype=torch.bfloat16, tensors=None) -> Path:
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file(tensors if tensors is not None else random_tensors(cfg, seed, dtype), str(path / "model.safetensors"))
    return path


def token_ids(vocab: int, n: int, seed: int) -> list:
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# ----------------------------------------------------------------------------- traces
def round64(n: int) -> int:
    return -(-n // 64) * 64


class TraceBuilder:
    """Collects steps and remembers, for each wanted logit row, which request and position it is."""

    def __init__(self):
        self.steps = []
        self.rows = {}  # step -> list of (request id, position)
        self._fed = {}

    def step(self, entries, end=()):
        """entries: list of (id, tokens, want)."""
        k = len(self.steps)
        rec = {"step": k, "entries": [], "end": list(end)}
        rows = []
        for rid, tokens, want in entries:
            base = self._fed.get(rid, 0)
            rec["entries"].append({"id": rid, "tokens": list(tokens), "want": list(want)})
            rows += [(rid, base + w) for w in want]
            self._fed[rid] = base + len(tokens)
        for rid in end:
            self._fed.pop(rid, None)
        self.steps.append(rec)
        if rows:
            self.rows[k] = rows
        return k


def run_trace(model_dir, dtype: str, steps, max_tokens: int, out_dir, timeout: int = 300, extra_env=None):
    """Run bin/trace_run on ``steps``; returns {step: float32 array [wanted, vocab]}."""
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens)]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    env = dict(os.environ)
    env.update(extra_env or {})
    proc = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=timeout, env=env)
    if proc.returncode != 0:
        raise AssertionError(f"trace_run failed ({proc.returncode}):\n{proc.stdout[-2000:]}\n{proc.stderr[-4000:]}")
    done = [line for line in proc.stdout.splitlines() if line.startswith("done ")]
    assert [d.split()[1] for d in done] == [str(s["step"]) for s in steps], "one 'done <step>' line per step, in order"
    vocab = json.loads((Path(model_dir) / "config.json").read_text())["vocab_size"]
    out = {}
    for s in steps:
        f = out_dir / f"{s['step']}.f32"
        wanted = sum(len(e["want"]) for e in s["entries"])
        if wanted:
            out[s["step"]] = np.fromfile(f, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not f.exists(), "no file for a step that wants nothing"
    return out


def collect(builder: TraceBuilder, results: dict) -> dict:
    """{request id: {position: logits row}} from a replay."""
    per = {}
    for step, rows in builder.rows.items():
        arr = results[step]
        for i, (rid, pos) in enumerate(rows):
            per.setdefault(rid, {})[pos] = arr[i]
    return per


# ----------------------------------------------------------------------------- comparison
F32_ATOL = 1e-4          # float32 engine against the plain implementation
BF16_REL = 2.0 ** -6     # bfloat16 engine: |diff| <= BF16_REL * max|plain logits of the sequence|


def assert_close_to_plain(got: np.ndarray, ref: np.ndarray, dtype: str, what: str):
    """Returns (rows whose plain logits have a clear winner, rows) for float32, where the argmax
    is compared on the clear rows; callers that check many rows sum them and require most to be
    clear, so that the argmax check is known to have had something to check."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    diff = np.abs(got - ref)
    tol = F32_ATOL if dtype == "float32" else BF16_REL * np.abs(ref).max()
    worst = np.unravel_index(diff.argmax(), diff.shape)
    assert diff.max() <= tol, (f"{what}: max|diff| {diff.max():.3e} > {tol:.3e} at row {worst[0]} "
                               f"(first wrong row: {int(np.argmax(diff.max(axis=-1) > tol))})")
    if dtype == "float32":
        # identical argmax wherever the plain logits have a clear winner
        top2 = np.sort(ref, axis=-1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 4 * F32_ATOL
        assert (got.argmax(-1)[clear] == ref.argmax(-1)[clear]).all(), f"{what}: argmax differs"
        return int(clear.sum()), int(clear.size)
    return 0, int(ref.shape[0])
