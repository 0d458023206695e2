"""Trace replay: feed given token ids through a model step by step and write logits.

The reference has no such program: its `replay` re-prints scheduler events
(flow_engine/cli.py:94-98) and its traces hold no token ids (trace.py:10). The
nearest behaviour is its test that feeds ids in portions through the forward
and compares logits (tests/test_engine.py:53-65). This program does that for
any script of steps. It samples nothing and owns no forward pass, cache or
loader: it drives the package's loader, cache manager and step function.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input: one JSON object per line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output: DIR/<step>.f32 (little-endian float32 [wanted, vocab]) for steps that
want logits, and a line `done <step>` on standard output after every step.
"""
from __future__ import annotations

import argparse
import json
import math
from pathlib import Path
import sys

PAGE_SIZE = 16
MAX_LIVE_REQUESTS = 64


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at once (each rounded up to a multiple of 64)")
    p.add_argument("--page-size", type=int, default=PAGE_SIZE,
                   help="tokens per cache page: any size the engine takes (a multiple of 4)")
    p.add_argument("--no-graphs", action="store_true", help="never replay decode steps from HIP graphs")
    return p.parse_args(argv)


def pool_pages(max_tokens, page_size):
    """Pages that hold MAX_TOKENS tokens of live requests, each request's count rounded up to a multiple of 64
    (of the page size, if that is larger): every 64 tokens of a request lie in at most ceil(64 / page) pages of
    its own, whatever the page size, so a page size that does not divide 64 gets the few pages more it needs."""
    if page_size >= 64:
        return math.ceil(max_tokens / page_size)
    return math.ceil(max_tokens / 64) * math.ceil(64 / page_size)


def run(args, lines, out=sys.stdout):
    import numpy as np
    import torch
    from ..cache import CacheManager
    from ..weights import load_model
    from .step import StepEntry, Stepper

    if args.max_tokens <= 0 or args.page_size <= 0 or args.page_size % 4:
        raise SystemExit("--max-tokens must be positive and --page-size a positive multiple of 4")
    if not torch.cuda.is_available():
        raise SystemExit("trace_run needs a GPU: there is no CPU path")
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    model = load_model(args.model, dtype=args.dtype, device="cuda:0")
    pages = pool_pages(args.max_tokens, args.page_size)
    cache = CacheManager(model.cache_layout(), args.page_size, pages, MAX_LIVE_REQUESTS, dtype=args.dtype,
                         device=model.device, prefix_cache=False,
                         max_request_tokens=pages * args.page_size)
    stepper = Stepper(model, cache, max_step_tokens=256, use_graphs=not args.no_graphs)
    live = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            seq = live.get(item["id"])
            if seq is None:
                seq = live[item["id"]] = cache.open(item["id"])
            entries.append(StepEntry(seq, list(item["tokens"]), list(item.get("want", []))))
        logits = stepper.step(entries)
        if logits.shape[0]:
            np.ascontiguousarray(logits.cpu().numpy(), dtype="<f4").tofile(str(out_dir / f"{step}.f32"))
        for rid in record.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                cache.close(seq)
        print(f"done {step}", file=out, flush=True)
    stepper.close()
    return 0


def main(argv=None):
    args = parse_args(argv)
    return run(args, sys.stdin)


if __name__ == "__main__":
    sys.exit(main())
