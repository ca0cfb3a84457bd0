"""Trace replay: feed given token ids through the model step by step and write the logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the same
``Model`` and ``Runner`` (step function, cache manager, kernels) that generation uses.

Input, one JSON object a line on standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one batch.  For a step that wants logits, ``<out>/<step>.f32`` holds
them as little-endian float32 [wanted, vocab] in the order of the entries and of ``want``.
After every step a line ``done <step>`` is printed and flushed.  When the input ends,
``<out>/cache_stats.json`` says how many pages each group's pool has, how often a page was handed
out, and how many pages were handed out more than once.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PAGE_SIZE = 16
MAX_LIVE_REQUESTS = 16


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to 64)")
    parser.add_argument("--page-size", type=int, default=PAGE_SIZE)
    args = parser.parse_args(argv)

    print("[trace_run] loading the kernel library and the model", file=sys.stderr, flush=True)
    import numpy as np
    import torch

    from .. import ops
    from .context import StepEntry
    from .model import Model, Runner

    ops.load()
    model = Model.from_pretrained(args.model, dtype=args.dtype, device="cuda:0")
    page = max(1, args.page_size)
    num_pages = -(-max(args.max_tokens, 64) // page)
    runner = Runner(model, page_size=page, num_pages=num_pages, max_requests=MAX_LIVE_REQUESTS)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    print(f"[trace_run] ready: {args.dtype}, {num_pages} pages of {page} tokens", file=sys.stderr, flush=True)

    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in live:
                live[rid] = runner.manager.open(rid)
            entries.append(StepEntry(live[rid], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                arr = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                arr.tofile(out_dir / f"{step}.f32")
            else:
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if rid in live:
                runner.manager.close(live.pop(rid))
        print(f"done {step}", flush=True)
    # what the cache manager did, for whoever wants to check that pages were used again
    stats = {"page_size": page, "groups": [
        {"pages": a.num_pages, "pages_issued": a.pages_issued, "pages_issued_again": len(a.pages_issued_again()),
         "free_at_end": a.num_free} for a in runner.manager.allocators],
        "steps": runner.steps, "tokens": runner.tokens}
    (out_dir / "cache_stats.json").write_text(json.dumps(stats) + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
