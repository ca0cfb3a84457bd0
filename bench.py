"""Decode and prefill throughput at Qwen2.5-7B shape with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch through the engine (scheduler, step function,
sampling).  The default run has the layer sizes of BASELINE.json's configs[2], a batch of 8
requests with 512-token prompts, and times K decode steps after W warm-up steps.  One JSON line
is printed: decoded tokens a second, the prefill of 2,048 tokens, the decode step against the
HBM roofline, and decode at batch 1 and 64.
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# published MI355X peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN25_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 3584,
    "num_hidden_layers": 28, "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "use_sliding_window": False,
}


# the other shapes that BASELINE.json lists (configs[3] and [4]); the default run is configs[2]
QWEN25_14B = dict(QWEN25_7B, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40, num_key_value_heads=8,
                  intermediate_size=13824, rms_norm_eps=1e-5, max_position_embeddings=8192)
QWEN25_32B = dict(QWEN25_14B, num_hidden_layers=64, intermediate_size=27648, max_position_embeddings=16384)
# the size the reference's own benchmarks run (README.md:39-48 there): Qwen2.5-0.5B, tied embeddings
QWEN25_05B = dict(QWEN25_7B, hidden_size=896, num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2, head_dim=64,
                  intermediate_size=4864, vocab_size=151936, tie_word_embeddings=True, max_position_embeddings=32768)
SHAPES = {"0.5b": ("Qwen2.5-0.5B shape", QWEN25_05B), "7b": ("Qwen2.5-7B shape", QWEN25_7B),
          "14b": ("Qwen2.5-14B shape", QWEN25_14B), "32b": ("Qwen2.5-32B shape", QWEN25_32B)}


def gemm_params_per_layer(c) -> int:
    q, kv = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    return c.hidden_size * (q + 2 * kv) + q * c.hidden_size + 3 * c.hidden_size * c.intermediate_size


def prefill_flops(c, layers: int, tokens: int) -> float:
    gemm = 2.0 * tokens * gemm_params_per_layer(c) * layers + 2.0 * c.hidden_size * c.vocab_size
    attn = 2.0 * c.num_attention_heads * c.head_dim * tokens * tokens * layers  # QK^T and PV, causal half
    return gemm + attn


def decode_bytes(c, layers: int, batch: int, context: float, itemsize: int) -> float:
    """Every weight the step uses once, and the cache of the live requests."""
    weights = (gemm_params_per_layer(c) * layers + c.hidden_size * c.vocab_size) * itemsize
    q = c.num_attention_heads * c.head_dim
    weights += (2 * c.hidden_size + q + 2 * c.num_key_value_heads * c.head_dim) * 4 * layers  # norms, biases (fp32)
    cache = batch * context * 2 * c.num_key_value_heads * c.head_dim * itemsize * layers
    return weights + cache


def other_workload(args, cfg, model, shape_name, layers, full_layers, page) -> int:
    """The two workloads of BASELINE.json beside the default run; one JSON line each."""
    import torch

    from from_scratch_inference_engine_amd import Engine, SamplingParams

    gen = torch.Generator().manual_seed(0)
    budget = 2048
    base = {"unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": args.dtype,
            "data": "synthetic: random weights N(0,0.02), uniform random token ids"}
    sizes = {"model": shape_name, "layers": layers, "layers_of_config": full_layers, "kv_block": page,
             "tokens_per_step": budget}
    if args.workload == "mixed":
        longest = args.max_prompt + args.outputs
        engine = Engine(model, block_size=page, num_blocks=args.requests * -(-longest // page) + 64,
                        max_batch=args.requests, max_tokens_per_step=budget)
        record = None
        # the same lengths in both passes: the first pays the graph captures and the library's kernel
        # selection for every step size they lead to, the second is measured
        lens = torch.randint(args.min_prompt, args.max_prompt + 1, (args.requests,), generator=gen).tolist()
        for rep in range(2):
            prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lens]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ids = [engine.add_request(p, SamplingParams(temperature=0.0), max_tokens=args.outputs) for p in prompts]
            first = None
            while engine.has_work():
                engine.step()
                if first is None and all(len(engine.output(i)) > 0 for i in ids):
                    torch.cuda.synchronize()
                    first = time.perf_counter() - t0
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            made = sum(len(engine.output(i)) for i in ids)
            print(f"[bench] pass {rep}: {sum(lens)} prompt tokens, {made} generated in {dt * 1e3:.0f} ms "
                  f"({first * 1e3:.0f} ms until every request had a token)", file=sys.stderr, flush=True)
            record = {"metric": f"tokens/s (prompt + generated) of {args.requests} requests through the scheduler, {shape_name}",
                      "value": (sum(lens) + made) / dt, "generated_per_s": made / dt, "ms": dt * 1e3,
                      "ms_until_all_started": first * 1e3, "prompt_tokens": sum(lens), "generated_tokens": made,
                      "config": dict(sizes, requests=args.requests, min_prompt=args.min_prompt,
                                     max_prompt=args.max_prompt, outputs=args.outputs)}
        print(json.dumps(dict(base, **record)))
        return 0
    n = args.prefill_tokens
    engine = Engine(model, block_size=page, num_blocks=-(-(n + 1) // page) + 64, max_batch=1,
                    max_tokens_per_step=budget)
    times = []
    for rep in range(3):
        prompt = torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.generate(prompt, SamplingParams(temperature=0.0), max_tokens=1)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        print(f"[bench] prefill of {n} tokens, pass {rep}: {times[-1] * 1e3:.0f} ms", file=sys.stderr, flush=True)
    dt = min(times[1:])
    print(json.dumps(dict(base, metric=f"prefill tokens/s, one prompt of {n} tokens in portions of {budget}, {shape_name}",
                          value=n / dt, ms=dt * 1e3, frac=prefill_flops(cfg, layers, n) / dt / PEAK_FLOPS[args.dtype],
                          config=dict(sizes, prefill_tokens=n))))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration (named in config)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="7b", help="layer sizes (default: BASELINE.json's configs[2])")
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--no-tune", action="store_true", help="leave the library's kernel choice for prefill to its heuristic")
    ap.add_argument("--workload", choices=["decode", "mixed", "long-prefill"], default="decode",
                    help="decode: the default run.  mixed: --requests prompts of --min-prompt to --max-prompt tokens, "
                         "--outputs tokens each, through the scheduler (BASELINE.json's configs[3] with --shape 14b).  "
                         "long-prefill: one prompt of --prefill-tokens tokens in portions of the token budget "
                         "(configs[4] with --shape 32b)")
    ap.add_argument("--requests", type=int, default=32)
    ap.add_argument("--min-prompt", type=int, default=128)
    ap.add_argument("--max-prompt", type=int, default=4096)
    ap.add_argument("--outputs", type=int, default=128)
    ap.add_argument("--prefill-tokens", type=int, default=16384)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import torch

    from from_scratch_inference_engine_amd import Engine, SamplingParams
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Model
    from from_scratch_inference_engine_amd.models import parse_config
    from from_scratch_inference_engine_amd.ops import enable_library_tuning

    if not args.no_tune and args.dtype == "bf16":
        enable_library_tuning()  # the first prefill times the library's kernels for its shapes

    shape_name, shape = SHAPES[args.shape]
    raw = dict(shape)
    full_layers = raw["num_hidden_layers"]
    layers = args.layers or full_layers
    raw["num_hidden_layers"] = layers
    cfg = parse_config(raw)
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    itemsize = 2 if args.dtype == "bf16" else 4
    t0 = time.perf_counter()
    model = Model.from_random(cfg, seed=0, dtype=dtype)
    torch.cuda.synchronize()
    print(f"[bench] {layers}-layer model with random weights on the GPU: {model.weight_bytes / 1e9:.2f} GB "
          f"in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)

    page = 16
    context = raw["max_position_embeddings"]
    if args.workload != "decode":
        return other_workload(args, cfg, model, shape_name, layers, full_layers, page)
    biggest = max(args.batch, 1 if args.no_points else 64)
    budget = 2048  # tokens a step may hold: the prompts of a large batch enter over several steps
    # requests whose prompt went in first decode while the others' prompts still enter: they get
    # that many more tokens, so that nobody ends inside the timed steps
    head_start = -(-biggest * args.prompt_len // budget) + 1
    per_req = args.prompt_len + args.steps + args.warmup + head_start + 2 * page
    num_blocks = max(biggest * -(-per_req // page), -(-2048 // page) * 2) + 64
    engine = Engine(model, block_size=page, num_blocks=num_blocks, max_batch=biggest, max_tokens_per_step=budget)
    gen = torch.Generator().manual_seed(0)

    def prompts(n, length):
        return [torch.randint(0, cfg.vocab_size, (length,), generator=gen).tolist() for _ in range(n)]

    # ---- prefill of 2,048 tokens: one request, one step
    runner = engine.runner
    pre_tokens = 2048
    times = []
    for rep in range(3):
        rc = runner.manager.open(f"prefill{rep}")
        ids = prompts(1, pre_tokens)[0]
        torch.cuda.synchronize()
        t = time.perf_counter()
        runner.step([StepEntry(rc, ids, [pre_tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
        runner.manager.close(rc)
        if rep == 0:
            print(f"[bench] first prefill (kernel selection, first launches): {times[0]:.1f} s", file=sys.stderr, flush=True)
    pre_s = min(times[1:])
    prefill = {"value": pre_tokens / pre_s, "tokens": pre_tokens, "ms": pre_s * 1e3,
               "frac": prefill_flops(cfg, layers, pre_tokens) / pre_s / PEAK_FLOPS[args.dtype]}
    print(f"[bench] prefill {pre_tokens} tokens: {pre_s * 1e3:.1f} ms", file=sys.stderr, flush=True)

    # ---- decode
    def decode(batch, steps, warmup):
        ids = [engine.add_request(p, SamplingParams(temperature=0.0), max_tokens=steps + warmup + head_start + 1)
               for p in prompts(batch, args.prompt_len)]
        while any(len(engine.output(i)) == 0 for i in ids):  # prompts in portions of the token budget
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        mean_ctx = args.prompt_len + 1 + warmup + steps / 2.0
        while engine.has_work():
            engine.step()
        return dt, mean_ctx

    dt, mean_ctx = decode(args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / dt
    step_bytes = decode_bytes(cfg, layers, args.batch, mean_ctx, itemsize)
    achieved = step_bytes / (dt / args.steps) / 1e9
    print(f"[bench] decode batch {args.batch}: {dt / args.steps * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            k = min(args.steps, 64)
            d, _ = decode(b, k, min(args.warmup, 16))
            points[f"decode_b{b}"] = b * k / d
            print(f"[bench] decode batch {b}: {d / k * 1e3:.3f} ms/step", file=sys.stderr, flush=True)

    line = {
        "metric": f"decode tok/s @ batch {args.batch}, {shape_name} (with prefill tok/s @ 2,048 tokens, decode @ batch 1/64)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0,0.02), uniform random token ids",
        "config": {
            "model": shape_name, "layers": layers, "layers_of_config": full_layers,
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": context, "prompt_len": args.prompt_len,
            "mean_decode_context": mean_ctx, "kv_block": page, "parallelism": "single GPU",
            "library_gemm_tuning": bool(not args.no_tune and args.dtype == "bf16"),
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": achieved / (HBM_BYTES_PER_S / 1e9)},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
