"""Command line: ``python -m from_scratch_inference_engine_amd <command>``.

Options keep the names the reference's harness uses (benchmarks/harness/bench_engine.py:118-131):
--model-dir, --num-requests, --prompt, --max-tokens, --block-size, --num-blocks, --temperature,
--json; the model folder defaults to $ENGINE_MODEL_DIR.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from time import perf_counter


def _common(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model-dir", default=os.environ.get("ENGINE_MODEL_DIR"),
                   help="folder with config.json and model.safetensors (default: $ENGINE_MODEL_DIR)")
    p.add_argument("--config", default=None, help="a config.json, with --random-weights: a model without a folder")
    p.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                   help="with --config: random weights made on the device from this seed")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--num-blocks", type=int, default=2048,
                   help="pages in the cache pool (0: as many as the free device memory holds)")
    p.add_argument("--max-batch", type=int, default=256)
    p.add_argument("--max-tokens-per-step", type=int, default=2048)
    p.add_argument("--prefill-chunk", type=int, default=None,
                   help="longest portion of a prompt in one step (default: the step's token budget)")
    p.add_argument("--max-tokens", type=int, default=64)
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-k", type=int, default=0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--tune-gemms", action="store_true",
                   help="time the library's kernels for the prefill products once per shape (seconds) and keep the best")
    p.add_argument("--no-weight-copies", action="store_true",
                   help="do not keep the large matrices a second time in the order the decode kernels read them "
                        "(half the memory, decode steps some 8 %% slower)")
    p.add_argument("--json", action="store_true", help="emit results as JSON")


def _llm(args):
    from .llm import LLM

    if args.config is not None or args.random_weights is not None:
        if args.config is None or args.random_weights is None:
            raise SystemExit("--config FILE and --random-weights SEED go together")
        with open(args.config) as f:
            raw = json.load(f)
        return LLM.from_config(raw, args.random_weights, block_size=args.block_size, num_blocks=args.num_blocks,
                               seed=args.seed, max_batch=args.max_batch, dtype=args.dtype,
                               max_tokens_per_step=args.max_tokens_per_step, prefill_chunk=args.prefill_chunk,
                               weight_copies=not args.no_weight_copies, tune_gemms=args.tune_gemms)
    if not args.model_dir:
        raise SystemExit("--model-dir (or $ENGINE_MODEL_DIR), or --config with --random-weights, is required")
    return LLM(args.model_dir, block_size=args.block_size, num_blocks=args.num_blocks, seed=args.seed,
               max_batch=args.max_batch, dtype=args.dtype, max_tokens_per_step=args.max_tokens_per_step,
               prefill_chunk=args.prefill_chunk, tune_gemms=args.tune_gemms, weight_copies=not args.no_weight_copies)


def _prompts(args, llm):
    if args.prompt_ids:
        return [[int(t) for t in spec.replace(",", " ").split()] for spec in args.prompt_ids]
    if args.prompt is not None:
        return [llm.tokenizer.encode(args.prompt)]
    raise SystemExit("give --prompt TEXT (needs tokenizer.json) or --prompt-ids '1 2 3'")


def cmd_generate(args) -> int:
    from .llm import GenerationConfig

    llm = _llm(args)
    cfg = GenerationConfig(args.max_tokens, args.temperature, args.top_k, args.top_p)
    prompts = _prompts(args, llm)
    outs = llm.generate_ids_batch(prompts, cfg)
    if args.json:
        print(json.dumps({"prompts": prompts, "outputs": outs}))
    else:
        for p, o in zip(prompts, outs):
            if args.prompt is not None and not args.prompt_ids:
                print(llm.tokenizer.decode(o))
            else:
                print(" ".join(map(str, o)))
    return 0


def cmd_bench(args) -> int:
    """Submit --num-requests copies of the prompt at once and report TTFT, TPOT and throughput
    (the reference's bench_engine.py:48-116)."""
    import statistics

    from ..sampling.params import SamplingParams
    from .scheduler import SeqStatus

    llm = _llm(args)
    prompt = _prompts(args, llm)[0]
    engine = llm.engine
    params = SamplingParams(args.temperature, args.top_k, args.top_p)
    start = perf_counter()
    ids = [engine.add_request(prompt, params, args.max_tokens, llm.eos_id) for _ in range(args.num_requests)]
    first, done, count = {}, {}, {}
    while engine.has_work():
        engine.step()
        now = perf_counter()
        for i in ids:
            if i not in first and engine.output(i):
                first[i] = now
            if i not in done and engine.status(i) == SeqStatus.Finished:
                done[i] = now
                count[i] = len(engine.output(i))
    wall = perf_counter() - start
    ttft = [(first[i] - start) * 1e3 for i in ids]
    tpot = [(done[i] - first[i]) * 1e3 / (count[i] - 1) for i in ids if count[i] > 1]
    total = sum(count.values())
    result = {
        "requests": len(ids), "prompt_tokens": len(prompt), "max_tokens": args.max_tokens,
        "total_output_tokens": total, "wall_seconds": wall,
        "throughput_tokens_per_s": total / wall if wall > 0 else 0.0,
        "requests_per_s": len(ids) / wall if wall > 0 else 0.0,
        "ttft_ms_mean": statistics.fmean(ttft), "ttft_ms_p50": sorted(ttft)[len(ttft) // 2],
        "ttft_ms_p90": sorted(ttft)[min(len(ttft) - 1, int(round(0.9 * (len(ttft) - 1))))],
        "tpot_ms_mean": statistics.fmean(tpot) if tpot else 0.0, "preemptions": engine.preemptions(),
    }
    if args.json:
        print(json.dumps(result, indent=2))
    else:
        for k, v in result.items():
            print(f"{k + ':':28s}{v:.3f}" if isinstance(v, float) else f"{k + ':':28s}{v}")
    return 0


def cmd_random_model(args) -> int:
    import torch

    from ..models.registry import parse_config
    from ..weights.random_init import write_random_model

    raw = json.loads(open(args.config, encoding="utf-8").read())
    out = write_random_model(parse_config(raw), args.seed, args.out,
                             torch.float32 if args.dtype == "float32" else torch.bfloat16)
    print(out)
    return 0


def cmd_replay(args) -> int:
    from .replay import main as replay_main

    return replay_main(args.rest)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="from_scratch_inference_engine_amd", description=__doc__)
    sub = parser.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="generate from token ids or text")
    _common(g)
    g.add_argument("--prompt", default=None)
    g.add_argument("--prompt-ids", action="append", help="token ids, e.g. '1 5 2 8' (repeat for a batch)")
    g.set_defaults(fn=cmd_generate)
    b = sub.add_parser("bench", help="batch-submitted latency/throughput benchmark")
    _common(b)
    b.add_argument("--num-requests", type=int, default=8)
    b.add_argument("--prompt", default=None)
    b.add_argument("--prompt-ids", action="append")
    b.set_defaults(fn=cmd_bench)
    r = sub.add_parser("random-model", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    r.set_defaults(fn=cmd_random_model)
    t = sub.add_parser("replay", help="trace replay (same as bin/trace_run)")
    t.add_argument("rest", nargs=argparse.REMAINDER)
    t.set_defaults(fn=cmd_replay)
    args = parser.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
