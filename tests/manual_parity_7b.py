"""Float32 parity of the engine with the plain implementation at Qwen2.5-7B shape.

Not collected by pytest (it needs about 35 GB of host memory, 30 GB of GPU memory and a few
minutes): run it by hand on the GPU box,

    python tests/manual_parity_7b.py [--layers 28] [--tokens 96]

It writes a model folder with random weights (bfloat16 values, so that both sides read the same
numbers), runs the plain implementation on the CPU for a few prompts, and the engine in float32 on
the GPU with the same prompts whole, with the last tokens decoded one by one, in portions, and
mixed in one batch.  Prints the largest absolute difference of the logits and whether every
argmax agrees; exits 1 if a difference exceeds 1e-4.
"""

from __future__ import annotations

import argparse
import sys
import tempfile
import time
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import plain_qwen2 as plain  # noqa: E402


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=28)
    ap.add_argument("--tokens", type=int, default=96)
    args = ap.parse_args()

    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Model, Runner
    from from_scratch_inference_engine_amd.models import parse_config
    from from_scratch_inference_engine_amd.weights import write_random_model

    raw = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 3584,
           "num_hidden_layers": args.layers, "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128,
           "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": False, "max_position_embeddings": 4096}
    with tempfile.TemporaryDirectory() as d:
        t0 = time.time()
        write_random_model(parse_config(raw), 0, d, torch.bfloat16)
        print(f"model folder written in {time.time() - t0:.0f} s", flush=True)
        cfg, w = plain.read_config(d), plain.read_weights(d)
        g = torch.Generator().manual_seed(0)
        lengths = [args.tokens, args.tokens // 2 + 3, 17]
        prompts = [torch.randint(0, 152064, (n,), generator=g).tolist() for n in lengths]
        t0 = time.time()
        ref = [plain.forward(cfg, w, p) for p in prompts]
        print(f"plain implementation: {time.time() - t0:.0f} s", flush=True)
        # the same with every matrix product in float64: how far float32 products alone move the logits
        linear32 = plain.linear
        plain.linear = lambda x, wt, b=None: (x.double() @ wt.double().t() + (0 if b is None else b.double())).float()
        ref64 = plain.forward(cfg, w, prompts[2])
        plain.linear = linear32
        print(f"plain float32 products against float64 products (17 tokens): max|diff| "
              f"{(ref[2] - ref64).abs().max().item():.3e}", flush=True)
        # the plain model with activations rounded to bfloat16 where the bfloat16 engine rounds
        # them (the inputs of every product, q/k/v after rotation, the gated activations):
        # what rounding alone does to the logits, for the bfloat16 pass below
        r16 = lambda t: t.to(torch.bfloat16).float()
        plain.linear = lambda x, wt, b=None: linear32(r16(x), wt, b)
        rope32, silu32 = plain.rope, plain.silu_mul
        plain.rope = lambda *a, **k: r16(rope32(*a, **k))
        plain.silu_mul = lambda g, u: r16(silu32(r16(g), r16(u)))
        ref16 = [plain.forward(cfg, w, p) for p in prompts]
        plain.linear, plain.rope, plain.silu_mul = linear32, rope32, silu32
        for i in range(len(prompts)):
            print(f"plain with bfloat16-rounded activations against plain, prompt {i}: max|diff| / max|logit| "
                  f"{((ref16[i] - ref[i]).abs().max() / ref[i].abs().max()).item():.3e}", flush=True)
        del w
        model = Model.from_pretrained(d, dtype="float32")
        runner = Runner(model, page_size=16, num_pages=64, max_requests=4)

        def run(plan):
            """plan: list of steps, each a list of (prompt index, n tokens)."""
            caches, fed = {}, {i: 0 for i in range(len(prompts))}
            rows = {i: [] for i in range(len(prompts))}
            for step in plan:
                entries = []
                for i, n in step:
                    if i not in caches:
                        caches[i] = runner.manager.open(f"r{i}")
                    entries.append(StepEntry(caches[i], prompts[i][fed[i]:fed[i] + n], list(range(n))))
                    fed[i] += n
                out = runner.step(entries).cpu()
                at = 0
                for (i, n) in step:
                    rows[i].append(out[at:at + n])
                    at += n
            for c in caches.values():
                runner.manager.close(c)
            return {i: torch.cat(r) for i, r in rows.items() if r}

        ways = {
            "whole": [[(i, len(p))] for i, p in enumerate(prompts)],
            "last 16 decoded": sum(([[(i, len(p) - 16)]] + [[(i, 1)] for _ in range(16)] for i, p in enumerate(prompts)), []),
            "portions": [[(0, 7)], [(0, 2)], [(0, 33)], [(0, args.tokens - 42)]],
            "mixed": [[(0, 40), (1, 5)], [(0, 1), (1, 20), (2, 17)], [(0, args.tokens - 41), (1, len(prompts[1]) - 25)]],
        }
        worst = 0.0
        for name, plan in ways.items():
            got = run(plan)
            for i, logits in got.items():
                diff = (logits - ref[i]).abs().max().item()
                same = bool((logits.argmax(-1) == ref[i].argmax(-1)).all())
                worst = max(worst, diff)
                note = f"  against float64 products {(logits - ref64).abs().max().item():.3e}" if i == 2 else ""
                print(f"{name:16s} prompt {i} ({len(prompts[i])} tokens): max|diff| {diff:.3e}  argmax identical: {same}{note}",
                      flush=True)
                if not same:
                    worst = max(worst, 1.0)
        print(f"largest difference {worst:.3e} (limit 1e-4)")
        if worst > 1e-4:
            return 1
        # the bfloat16 engine on the same weights: reported against the plain float32 logits in
        # units of their largest magnitude (the tests' bound at tiny sizes is 2^-6), and how often
        # it picks the plain model's token where that one leads by more than the difference
        del runner, model
        torch.cuda.empty_cache()
        model = Model.from_pretrained(d, dtype="bfloat16")
        runner = Runner(model, page_size=16, num_pages=64, max_requests=4)
        worst_rel, wrong = 0.0, 0
        for name in ("whole", "last 16 decoded", "mixed"):
            got = run(ways[name])
            for i, logits in got.items():
                scale = ref[i].abs().max().item()
                rel = (logits - ref[i]).abs().max().item() / scale
                rel16 = (logits - ref16[i]).abs().max().item() / scale
                top2 = ref[i].topk(2, dim=-1).values
                clear = (top2[:, 0] - top2[:, 1]) > 2 * rel * scale
                agree = (logits.argmax(-1) == ref[i].argmax(-1))[clear].float().mean().item() if clear.any() else 1.0
                worst_rel = max(worst_rel, rel)
                print(f"bfloat16 {name:16s} prompt {i}: max|diff| / max|logit| {rel:.3e} (against the rounded plain model "
                      f"{rel16:.3e})  argmax agrees where clear: {agree:.3f} ({int(clear.sum())} of {clear.numel()} rows clear)",
                      flush=True)
                wrong += int(((logits.argmax(-1) != ref[i].argmax(-1)) & clear).sum())
        print(f"bfloat16: largest relative difference {worst_rel:.3e}; rows with a clear plain choice that the engine "
              f"does not share: {wrong}")
        return 0 if wrong == 0 else 1


if __name__ == "__main__":
    sys.exit(main())
