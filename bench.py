"""Decode and prefill throughput at Qwen2.5-7B shape with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch through the engine (scheduler, step function,
sampling).  The default run has 28 layers of hidden 3584 / intermediate 18944 with 28 query and 4
key/value heads of 128 and a vocabulary of 152,064, a batch of 8 requests with 512-token prompts,
and times K decode steps after W warm-up steps.  One JSON line is printed: decoded tokens a
second, the prefill of 2,048 tokens, the decode step against the HBM roofline, decode at batch 1
and 64, and the time of each class of kernels of a decode step.
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


# the two larger shapes: 48 layers of 5120 / 13824 and 64 layers of 5120 / 27648, 40 query and 8 key/value heads
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


def kernel_classes(runner, cfg, batch: int, prompt_len: int, itemsize: int) -> dict:
    """Time of each class of kernels of one decode step: the calls of an eagerly run step are
    recorded (kernel, operands), and each class's calls, over all layers with each layer's own
    weights, are captured into a graph of their own and timed with events around its replays.
    GB/s = the weights (for attention: the live cache) the class reads once a step / its time."""
    import torch

    from from_scratch_inference_engine_amd import ops
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.parts import linear as linear_module

    h, inter, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    q = cfg.num_attention_heads * cfg.head_dim

    def matrix_class(w):
        n, k = w.shape
        if n == v:
            return "lm_head"
        if n == 2 * inter:
            return "gate_up"
        if k == inter:
            return "down"
        if n == q + 2 * cfg.num_key_value_heads * cfg.head_dim:
            return "qkv"
        return "o" if (n, k) == (h, q) else "other"

    classify = {
        "gemm_mfma_skinny_rope": lambda a, k: "qkv", "rope_kv_write": lambda a, k: "qkv", "bias_add": lambda a, k: "qkv",
        "attention_mfma": lambda a, k: "attention", "attention_mfma_lds": lambda a, k: "attention",
        "attention_mfma_qkv": lambda a, k: "attention",
        "attention_scalar": lambda a, k: "attention", "attention_merge": lambda a, k: "attention",
        "gemm_mfma_skinny": lambda a, k: matrix_class(a[1]), "gemm_mfma_wide": lambda a, k: matrix_class(a[1]),
        "gemm_mfma_wide_swiglu": lambda a, k: "gate_up",
        "gemm": lambda a, k: matrix_class(a[1]), "gemm_mfma_fp32": lambda a, k: matrix_class(a[1]),
        "library_mm": lambda a, k: matrix_class(a[1]),
        "swiglu": lambda a, k: "gate_up", "rmsnorm": lambda a, k: "norms", "embedding": lambda a, k: "other",
        "rope_table": lambda a, k: "other", "residual_add": lambda a, k: "other",
    }
    calls = []
    saved = {name: getattr(ops, name) for name in classify}
    saved_mm = linear_module.library_mm

    def recorder(name, fn):
        def run(*a, **k):
            calls.append((classify[name](a, k), fn, a, k))
            return fn(*a, **k)
        return run

    gen = torch.Generator().manual_seed(1)
    caches = [runner.manager.open(f"classes{i}") for i in range(batch)]
    graphs, runner.graphs = runner.graphs, None
    try:
        for c in caches:  # their prompts, then one decode step with the recorder on
            runner.step([StepEntry(c, torch.randint(0, v, (prompt_len,), generator=gen).tolist(), [])])
        for name, fn in saved.items():
            setattr(ops, name, recorder(name, fn))
        linear_module.library_mm = recorder("library_mm", saved_mm)
        runner.step([StepEntry(c, [7], [0]) for c in caches])
    finally:
        for name, fn in saved.items():
            setattr(ops, name, fn)
        linear_module.library_mm = saved_mm
        runner.graphs = graphs
    weights = {"qkv": h * (q + 2 * cfg.num_key_value_heads * cfg.head_dim), "o": q * h, "gate_up": 2 * h * inter,
               "down": h * inter}
    n_layers = sum(1 for c in calls if c[0] == "down")  # (one product a layer, whichever kernel takes it)
    read = {k: n * itemsize * n_layers for k, n in weights.items()}
    read["lm_head"] = h * v * itemsize
    read["attention"] = batch * (prompt_len + 1) * 2 * cfg.num_key_value_heads * cfg.head_dim * itemsize * n_layers
    out = {}
    # The recorded step and the prompts before it are only queued so far.  Every call below reads that
    # step's tables and intermediate tensors, so they must be complete first; and the calls run on the
    # stream that filled them, never on another one that would not wait for it.
    torch.cuda.synchronize()
    for cls in sorted({c[0] for c in calls}):
        mine = [(fn, a, k) for c, fn, a, k in calls if c == cls]
        for fn, a, k in mine:  # once outside a capture: first launches, the allocator's blocks
            fn(*a, **k)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for fn, a, k in mine:
                fn(*a, **k)
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 10
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out[cls] = {"ms": round(ms, 4), "launches": len(mine)}
        if cls in read:
            out[cls]["GB/s"] = round(read[cls] / ms / 1e6, 1)
        del graph
    for c in caches:
        runner.manager.close(c)
    return out


def other_workload(args, cfg, model, shape_name, layers, full_layers, page, fill_rows) -> int:
    """The two workloads beside the default run (many requests of mixed lengths through the
    scheduler; one long prompt in portions); one JSON line each."""
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
                        max_batch=args.requests, max_tokens_per_step=budget, fill_rows=fill_rows)
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
                    max_tokens_per_step=budget, fill_rows=fill_rows)
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
    ap.add_argument("--shape", choices=sorted(SHAPES), default="7b", help="layer sizes (default: 28 layers of 3584 / 18944)")
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--max-positions", type=int, default=None,
                    help="position limit of the model (default: the shape's; raise it for prompts beyond that)")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--no-kernels", action="store_true", help="skip the time of each class of kernels of a decode step")
    ap.add_argument("--no-tune", action="store_true", help="leave the library's kernel choice for prefill to its heuristic")
    ap.add_argument("--no-streamed-copies", action="store_true",
                    help="do not keep the large weights a second time in the order of the matrix instruction's fragments")
    ap.add_argument("--workload", choices=["decode", "mixed", "long-prefill"], default="decode",
                    help="decode: the default run.  mixed: --requests prompts of --min-prompt to --max-prompt tokens, "
                         "--outputs tokens each, through the scheduler (made for --shape 14b).  "
                         "long-prefill: one prompt of --prefill-tokens tokens in portions of the token budget "
                         "(made for --shape 32b)")
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

    fill_rows = None
    if not args.no_tune and args.dtype == "bf16":
        from from_scratch_inference_engine_amd.engine.context import padded_tokens

        enable_library_tuning()  # the first prefill times the library's kernels for its shapes
        fill_rows = padded_tokens  # and steps that are not decode steps are filled up to the timed row counts

    shape_name, shape = SHAPES[args.shape]
    raw = dict(shape)
    full_layers = raw["num_hidden_layers"]
    layers = args.layers or full_layers
    raw["num_hidden_layers"] = layers
    if args.max_positions:
        raw["max_position_embeddings"] = args.max_positions
    cfg = parse_config(raw)
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    itemsize = 2 if args.dtype == "bf16" else 4
    t0 = time.perf_counter()
    model = Model.from_random(cfg, seed=0, dtype=dtype, weight_copies=not args.no_streamed_copies)
    torch.cuda.synchronize()
    print(f"[bench] {layers}-layer model with random weights on the GPU: {model.weight_bytes / 1e9:.2f} GB "
          f"in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)

    page = 16
    context = raw["max_position_embeddings"]
    if args.workload != "decode":
        return other_workload(args, cfg, model, shape_name, layers, full_layers, page, fill_rows)
    biggest = max(args.batch, 1 if args.no_points else 64)
    budget = 2048  # tokens a step may hold: the prompts of a large batch enter over several steps
    # requests whose prompt went in first decode while the others' prompts still enter: they get
    # that many more tokens, so that nobody ends inside the timed steps
    head_start = -(-biggest * args.prompt_len // budget) + 1
    per_req = args.prompt_len + args.steps + args.warmup + head_start + 2 * page
    num_blocks = max(biggest * -(-per_req // page), -(-2048 // page) * 2) + 64
    engine = Engine(model, block_size=page, num_blocks=num_blocks, max_batch=biggest, max_tokens_per_step=budget,
                    fill_rows=fill_rows)
    gen = torch.Generator().manual_seed(0)

    def prompts(n, length):
        return [torch.randint(0, cfg.vocab_size, (length,), generator=gen).tolist() for _ in range(n)]

    # ---- prefill of 2,048 tokens: one request, one step
    runner = engine.runner
    pre_tokens = 2048
    times = []
    for rep in range(6):  # the first one chooses kernels; the fastest of the other five counts
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
    points, points_frac = {}, {}
    if not args.no_points:
        for b in (1, 64):
            k = min(args.steps, 64)
            d, ctx_b = decode(b, k, min(args.warmup, 16))
            points[f"decode_b{b}"] = b * k / d
            # the same roofline fraction as for the timed batch: bytes of a step / its time / the peak
            points_frac[f"decode_b{b}"] = decode_bytes(cfg, layers, b, ctx_b, itemsize) / (d / k) / HBM_BYTES_PER_S
            print(f"[bench] decode batch {b}: {d / k * 1e3:.3f} ms/step", file=sys.stderr, flush=True)

    kernels = {}
    if not args.no_kernels:
        kernels = kernel_classes(runner, cfg, args.batch, args.prompt_len + args.warmup + args.steps // 2, itemsize)
        print("[bench] kernel classes of a decode step, ms: "
              + ", ".join(f"{k} {v['ms']:.3f}" for k, v in kernels.items()), file=sys.stderr, flush=True)

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
            "streamed_weight_copies": bool(not args.no_streamed_copies and args.dtype == "bf16"),
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": achieved / (HBM_BYTES_PER_S / 1e9)},
        "points": points,
        "points_roofline_frac": points_frac,
        "kernels": kernels,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
