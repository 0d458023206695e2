#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen2.5-7B shape on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Default run: the layer sizes of the 7B shape, random weights, bfloat16, a batch
of 8 requests decoding at a context of 4,096 tokens: each request is given a
random prompt of 4096 - W - K tokens, then W untimed and K timed decode steps
run through the scheduler (admission, planning, the step function, greedy
sampling on the device, commit), so the last timed step reads 4,096 keys per
request. One JSON line is printed: decoded tokens a second, a 2,048-token
prefill, the decode step's HBM roofline (against the nominal 8 TB/s and against
what a plain streaming reader reaches on this device, measured in the same run),
the library's rate on the prefill's matrix products (`prefill.library_gemm_tflops`; `frac_of_library` is the
whole step's rate against it), and further points: decode at batch 1, 16, 32 and 64 at the same context; the same batch
of 8 with the engine opened for 32,768 tokens a request (`decode_b8_open32k`)
and with requests of 16,384 tokens and of that length (`decode_b8_ctx16k`, `decode_b8_ctx32k`: the cache is then as large
as the weights; `prefill_32k_prompts`: tokens a second over those prompts, which
go through in portions of 2,048); and 1,024-token prompts with 512 generated tokens at batch 1, 8 and 64
(`gen512_b*`, decoded tokens a second over the generated part).

Other sizes of the architecture: --shape 14b|32b. --serve measures continuous
batching under Poisson arrivals instead (prompts of 128..4,096 tokens, 256
generated tokens each, prompt portions of 512) and prints its own JSON line.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

QWEN25_7B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=28, hidden_size=3584,
    num_attention_heads=28, num_key_value_heads=4, head_dim=128, intermediate_size=18944,
    vocab_size=152064, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False,
    use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu")

# Further shapes of the same architecture (--shape): sizes only, everything else as above.
SHAPES = {
    "0.5b": ("Qwen2.5-0.5B shape", dict(num_hidden_layers=24, hidden_size=896, num_attention_heads=14,
                                        num_key_value_heads=2, head_dim=64, intermediate_size=4864, vocab_size=151936,
                                        tie_word_embeddings=True)),
    "1.5b": ("Qwen2.5-1.5B shape", dict(num_hidden_layers=28, hidden_size=1536, num_attention_heads=12,
                                        num_key_value_heads=2, intermediate_size=8960, vocab_size=151936,
                                        tie_word_embeddings=True)),
    "3b": ("Qwen2.5-3B shape", dict(num_hidden_layers=36, hidden_size=2048, num_attention_heads=16,
                                    num_key_value_heads=2, intermediate_size=11008, vocab_size=151936,
                                    tie_word_embeddings=True)),
    "7b": ("Qwen2.5-7B shape", {}),
    "14b": ("Qwen2.5-14B shape", dict(num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
                                      num_key_value_heads=8, intermediate_size=13824, rms_norm_eps=1e-5)),
    "32b": ("Qwen2.5-32B shape", dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=40,
                                      num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-5)),
}

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=128)
    p.add_argument("--warmup", type=int, default=16)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=4096)
    p.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="layer sizes (default: the 7B shape)")
    p.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all of them)")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--points", default="1,16,32,64", help="further decode batch sizes to measure")
    p.add_argument("--max-context", type=int, default=0,
                   help="tokens a request may hold, which the engine is opened for (0: the context + 1)")
    p.add_argument("--no-extra-points", action="store_true",
                   help="skip decode_b8_open32k, decode_b8_ctx32k and the gen512_b* points (1,024-token prompts + 512 generated)")
    p.add_argument("--no-graphs", action="store_true")
    p.add_argument("--prefill-only", action="store_true", help="measure only the prefill (profiling runs)")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--yardstick", default="", help="rows, comma separated: time the four projections of a layer at these row "
                   "counts with this engine's kernels and with the library's (a table, no model is built)")
    p.add_argument("--serve", action="store_true",
                   help="instead: continuous batching of --requests requests (prompts of 128..4096 tokens, 256 "
                        "generated each, Poisson arrivals at --rate a second, prompt portions of 512)")
    p.add_argument("--requests", type=int, default=64)
    p.add_argument("--prefill-chunk", type=int, default=512,
                   help="with --serve: the largest prompt portion in one step (larger: more prompt tokens a second and "
                        "a shorter time to the first token, longer steps for the requests that are decoding)")
    p.add_argument("--rate", type=float, default=16.0, help="mean arrivals a second (0: all at once)")
    return p.parse_args()


def decode_run(model, torch, batch, context, steps, warmup, dtype, use_graphs, seed, max_context=0):
    """Tokens/s and ms/step of STEPS decode steps at BATCH, ending at CONTEXT keys per request; the graph
    replays; and the tokens a second at which the prompts went through beforehand (untimed for the former)."""
    from tessweave_engine_amd.config import EngineConfig
    from tessweave_engine_amd.engine import Engine

    prompt_len = context - steps - warmup
    assert prompt_len >= 1
    page = 16
    blocks = batch * ((context + page - 1) // page + 1)
    chunk = 2048
    config = EngineConfig(block_size=page, kv_blocks=blocks, max_context=max_context or context + 1, max_active=batch,
                          max_queue=batch, prefill_chunk=chunk, min_prefill_chunk=16, prefix_cache=False,
                          dtype=dtype, max_step_tokens=batch + chunk, use_graphs=use_graphs)
    engine = Engine(model, config)
    g = torch.Generator().manual_seed(seed)
    vocab = model.config.vocab_size
    requests = [engine.submit(torch.randint(0, vocab, (prompt_len,), generator=g).tolist(),
                              max_tokens=steps + warmup + 1, ignore_eos=True, stream=False) for _ in range(batch)]
    # Prompts, untimed: all but the last token of every prompt goes through the step function
    # directly, so that every request samples its first token in the same step and they decode in lockstep.
    from tessweave_engine_amd.engine import StepEntry
    engine._admit()
    assert len(engine.active) == batch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for r in requests:
        for i in range(0, prompt_len - 1, chunk):
            engine.stepper.step([StepEntry(r.seq, r.prompt[i:min(prompt_len - 1, i + chunk)], [])])
    torch.cuda.synchronize()
    prompt_tokens_per_s = batch * (prompt_len - 1) / (time.perf_counter() - t0)
    for _ in range(warmup):
        engine.step()
    engine.flush()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    engine.flush()                 # the last step's tokens are read inside the timed region too
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert all(len(r.output) == warmup + steps for r in requests), [len(r.output) for r in requests]
    replays = engine.stepper.graph_replays
    engine.close()
    del engine
    torch.cuda.empty_cache()
    return batch * steps / elapsed, elapsed / steps * 1000, replays, prompt_tokens_per_s


def serve_run(model, torch, args):
    """Continuous batching under arrivals: requests join while others decode; one JSON-ready dict."""
    from tessweave_engine_amd.config import EngineConfig
    from tessweave_engine_amd.engine import Engine

    page, chunk, outputs, longest = 16, args.prefill_chunk, 256, 4096
    n, active = args.requests, min(args.requests, 64)
    config = EngineConfig(block_size=page, kv_blocks=active * ((longest + outputs) // page + 1),
                          max_context=longest + outputs, max_active=active, max_queue=n, prefill_chunk=chunk,
                          min_prefill_chunk=16, prefix_cache=False, dtype=args.dtype,
                          max_step_tokens=active + chunk, use_graphs=not args.no_graphs)
    engine = Engine(model, config)
    g = torch.Generator().manual_seed(args.seed)
    lengths = torch.randint(128, longest + 1, (n,), generator=g).tolist()
    prompts = [torch.randint(0, model.config.vocab_size, (k,), generator=g).tolist() for k in lengths]
    gaps = torch.empty(n).exponential_(args.rate, generator=g).tolist() if args.rate > 0 else [0.0] * n
    arrivals, t = [], 0.0
    for gap in gaps:
        t += gap
        arrivals.append(t)
    engine.generate(prompts[:2], max_tokens=4, ignore_eos=True)          # untimed: first launches, workspace
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    requests, nxt, steps0 = [], 0, engine.stats()["steps"]
    while True:
        now = time.perf_counter() - t0
        while nxt < n and arrivals[nxt] <= now:
            requests.append(engine.submit(prompts[nxt], max_tokens=outputs, ignore_eos=True, stream=False))
            nxt += 1
        if engine.step():                       # False: nothing admitted and no token unread
            continue
        if nxt == n:
            break
        time.sleep(max(0.0, min(0.001, arrivals[nxt] - (time.perf_counter() - t0))))
    engine.flush()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert all(len(r.output) == outputs for r in requests), sorted(len(r.output) for r in requests)[:4]
    ttft = sorted((r.first_token - r.created) * 1000 for r in requests)
    stats = engine.stats()
    engine.close()
    generated, prompt_tokens = n * outputs, sum(lengths)
    return {"metric": "continuous batching, generated tokens a second", "value": round(generated / elapsed, 1),
            "unit": "tokens/s", "total_tokens_per_s": round((generated + prompt_tokens) / elapsed, 1),
            "seconds": round(elapsed, 3), "requests": n, "rate": args.rate, "prompt_tokens": prompt_tokens,
            "generated_tokens": generated, "ttft_ms_mean": round(sum(ttft) / n, 1),
            "ttft_ms_p50": round(ttft[n // 2], 1), "ttft_ms_p99": round(ttft[min(n - 1, int(n * 0.99))], 1),
            "steps": stats["steps"] - steps0, "graph_replays": stats["graph_replays"], "prefill_chunk": chunk,
            "max_active": active}


def read_ceiling(torch, device, gigabytes=4):
    """GB/s of a plain streaming reader (non-temporal 1 KB loads per wave, no arithmetic) over GIGABYTES of
    device memory: the read bandwidth this device gives a kernel that does nothing else."""
    from tessweave_engine_amd.kernels import ops
    buffer = torch.empty(gigabytes << 30, dtype=torch.uint8, device=device)
    buffer.zero_()
    out = torch.zeros(1, dtype=torch.float32, device=device)
    best = None
    for _ in range(5):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        n = ops.probe_read(buffer, out, blocks=4096)
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end)
        best = ms if best is None else min(best, ms)
    del buffer
    torch.cuda.empty_cache()
    return n / (best / 1000) / 1e9


def library_matrix_rate(torch, c, rows, layers, device, repeats=5):
    """TFLOP/s of the library's bfloat16 matrix product (hipBLASLt through torch.matmul) over the four projections
    of a layer at ROWS rows, LAYERS distinct weight sets in turn (so that, as in the model, weights come from HBM and
    not from a cache): the yardstick the prefill's own matrix kernels are measured against. Not on the product path."""
    qkv = (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim
    shapes = [(qkv, c.hidden_size), (c.hidden_size, c.num_attention_heads * c.head_dim),
              (2 * c.intermediate_size, c.hidden_size), (c.hidden_size, c.intermediate_size)]
    layers = max(1, min(layers, 4))
    weights = [[torch.randn(n, k, device=device, dtype=torch.bfloat16) * 0.02 for n, k in shapes] for _ in range(layers)]
    inputs = [torch.randn(rows, k, device=device, dtype=torch.bfloat16) for _, k in shapes]
    flops = layers * sum(2.0 * rows * n * k for n, k in shapes)
    best = None
    for i in range(repeats + 1):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for layer in weights:
            for x, w in zip(inputs, layer):
                torch.matmul(x, w.t())
        end.record()
        torch.cuda.synchronize()
        if i:
            ms = start.elapsed_time(end)
            best = ms if best is None else min(best, ms)
    del weights, inputs
    torch.cuda.empty_cache()
    return flops / (best / 1000) / 1e12


def yardstick_table(torch, c, rows_list, device, copies=4, repeats=5):
    """Microseconds and TFLOP/s of the four projections of a layer at each row count: this engine's kernels (shuffled
    weights, the choice `ops.linear` makes itself; gate_up with its SiLU-multiply epilogue) beside the library's
    bfloat16 product (hipBLASLt through torch.matmul; not on the product path). COPIES weight sets in turn, so that
    weights come from HBM as in the model."""
    from tessweave_engine_amd.kernels import ops
    qkv = (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim
    shapes = [("qkv", qkv, c.hidden_size, False), ("o", c.hidden_size, c.num_attention_heads * c.head_dim, False),
              ("gate_up", 2 * c.intermediate_size, c.hidden_size, True), ("down", c.hidden_size, c.intermediate_size, False)]
    lines = []
    for name, n, k, glu in shapes:
        plain = [torch.randn(n, k, device=device, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        shuffled = [ops.shuffle_weight(w) for w in plain]
        for rows in rows_list:
            x = torch.randn(rows, k, device=device, dtype=torch.bfloat16) * 0.1
            out = torch.empty(rows, n // 2 if glu else n, device=device, dtype=torch.bfloat16)
            work = torch.empty(max(ops.linear_workspace_bytes(torch.bfloat16, rows, n, k) // 4, 16), device=device)
            timed = {}
            engine = (lambda i: ops.linear_glu(x, shuffled[i], out)) if glu else \
                (lambda i: ops.linear(x, shuffled[i], out, workspace=work))
            for who, call in (("engine", engine),
                              ("library", lambda i: torch.matmul(x, plain[i].t()))):
                best = None
                for r in range(repeats + 1):
                    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    start.record()
                    for i in range(2 * copies):
                        call(i % copies)
                    end.record()
                    torch.cuda.synchronize()
                    if r:
                        us = start.elapsed_time(end) * 1000 / (2 * copies)
                        best = us if best is None else min(best, us)
                timed[who] = best
            flops = 2.0 * rows * n * k
            lines.append({"projection": name, "rows": rows, "n": n, "k": k,
                          "engine_us": round(timed["engine"], 1), "engine_tflops": round(flops / timed["engine"] / 1e6, 1),
                          "library_us": round(timed["library"], 1), "library_tflops": round(flops / timed["library"] / 1e6, 1)})
        del plain, shuffled
        torch.cuda.empty_cache()
    return lines


def prefill_run(model, torch, tokens, dtype, seed, repeats=3):
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper

    page = 16
    cache = CacheManager(model.cache_layout(), page, tokens // page + 2, 2, dtype=dtype, device=model.device,
                         prefix_cache=False, max_request_tokens=tokens + page)
    stepper = Stepper(model, cache, max_step_tokens=tokens, use_graphs=False)
    g = torch.Generator().manual_seed(seed + 1)
    ids = torch.randint(0, model.config.vocab_size, (tokens,), generator=g).tolist()
    best = None
    for i in range(repeats + 1):
        seq = cache.open(f"p{i}")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = stepper.step([StepEntry(seq, ids, [tokens - 1])])
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1000
        assert torch.isfinite(logits).all()
        cache.close(seq)
        if i > 0:
            best = ms if best is None else min(best, ms)
    stepper.close()
    return best


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine does not run on {args.gpus} GPUs")
        return 2
    import torch
    from tessweave_engine_amd.config import config_from_dict
    from tessweave_engine_amd.weights import random_model

    shape_name, sizes = SHAPES[args.shape]
    cfg = dict(QWEN25_7B, **sizes)
    layers_full = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    config = config_from_dict(cfg)
    if args.yardstick:
        for line in yardstick_table(torch, config, [int(v) for v in args.yardstick.split(",")], "cuda:0"):
            print(json.dumps(line))
        return 0
    model = random_model(config, args.seed, dtype=args.dtype, device="cuda:0")
    c = config
    use_graphs = not args.no_graphs

    if args.serve:
        line = serve_run(model, torch, args)
        line.update({"model": shape_name, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
                     "data": "synthetic: uniform-random token ids, random weights N(0, 0.02)"})
        print(json.dumps(line))
        return 0
    if args.prefill_only:
        ms = prefill_run(model, torch, args.prefill_tokens, args.dtype, args.seed)
        print(json.dumps({"prefill_ms": round(ms, 3), "tokens": args.prefill_tokens,
                          "tokens_per_s": round(args.prefill_tokens / (ms / 1000), 1)}))
        return 0
    value, ms_per_step, replays, _ = decode_run(model, torch, args.batch, args.context, args.steps, args.warmup,
                                             args.dtype, use_graphs, args.seed, args.max_context)
    element = 2 if args.dtype == "bfloat16" else 4
    layer_weights = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    weight_bytes = model.weight_bytes()          # what the model's parts say a step reads once in full
    assert abs(weight_bytes / ((c.num_hidden_layers * layer_weights + c.vocab_size * c.hidden_size) * element) - 1) < 2e-3
    mean_ctx = args.context - args.steps / 2
    kv_bytes = args.batch * mean_ctx * c.kv_bytes_per_token(element)
    achieved = (weight_bytes + kv_bytes) / (ms_per_step / 1000) / 1e9

    t = args.prefill_tokens
    if t <= 0:                      # decode only (profiling runs)
        print(json.dumps({"value": round(value, 1), "ms_per_step": round(ms_per_step, 4), "batch": args.batch,
                          "roofline_frac": round(achieved / HBM_PEAK_GBS, 4)}))
        return 0
    prefill_ms = prefill_run(model, torch, t, args.dtype, args.seed)
    linear_flops = 2.0 * t * c.num_hidden_layers * layer_weights + 2.0 * c.vocab_size * c.hidden_size
    attn_flops = c.num_hidden_layers * 4.0 * c.num_attention_heads * c.head_dim * (t * (t + 1) / 2)
    prefill_tflops = (linear_flops + attn_flops) / (prefill_ms / 1000) / 1e12

    # the library's rate on the same matrix products, and the engine's own rate on them if every other kernel of the
    # step took no time at all (a lower bound of what its matrix kernels reach)
    library = library_matrix_rate(torch, c, t, c.num_hidden_layers, model.device) if args.dtype == "bfloat16" else None

    points = {}
    for b in [int(v) for v in args.points.split(",") if v]:
        steps = min(args.steps, 64)
        tps, _, _, _ = decode_run(model, torch, b, args.context, steps, 8, args.dtype, use_graphs, args.seed,
                               args.max_context)
        points[f"decode_b{b}"] = round(tps, 1)
    if not args.no_extra_points:
        # the same batch with the engine opened for 32,768 tokens a request (launch shapes must follow the
        # lengths that are served, not the lengths that are allowed)
        opened = min(32768, c.max_position_embeddings)
        tps, _, _, _ = decode_run(model, torch, args.batch, args.context, min(args.steps, 64), 8, args.dtype, use_graphs,
                               args.seed, opened)
        points[f"decode_b{args.batch}_open{opened // 1024}k"] = round(tps, 1)
        # prompts of 1,024 tokens, 512 generated (8 of them untimed): decoded tokens a second over the rest
        for b in (1, 8, 64):
            tps, _, _, _ = decode_run(model, torch, b, 1024 + 512, 504, 8, args.dtype, use_graphs, args.seed, opened)
            points[f"gen512_b{b}"] = round(tps, 1)
        # a batch of 8 at half that length
        if opened >= 32768:
            tps, _, _, _ = decode_run(model, torch, args.batch, 16384, 32, 8, args.dtype, use_graphs, args.seed, opened)
            points[f"decode_b{args.batch}_ctx16k"] = round(tps, 1)
        # and with requests that really are that long: the cache is then as large as the weights
        tps, _, _, prompts_tps = decode_run(model, torch, args.batch, opened - 16, 32, 8, args.dtype, use_graphs, args.seed, opened)
        points[f"decode_b{args.batch}_ctx{opened // 1024}k"] = round(tps, 1)
        # what that run's prompts took: portions of 2,048 tokens, most of their keys from the cache
        points[f"prefill_{opened // 1024}k_prompts"] = round(prompts_tps, 1)
    ceiling = read_ceiling(torch, model.device)

    line = {
        "metric": f"decode tok/s @ batch {args.batch}, {shape_name} {'bf16' if args.dtype == 'bfloat16' else 'fp32'} "
                  f"(+ prefill tok/s @ {t}, decode @ batch {args.points or '-'})",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform-random token ids, random weights N(0, 0.02)",
        "config": {"model": shape_name, "layers": c.num_hidden_layers, "layers_full": layers_full,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": c.head_dim, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context,
                   "prompt_len": args.context - args.steps - args.warmup, "page_size": 16,
                   "parallelism": "single GPU", "hip_graphs": bool(use_graphs and replays > 0),
                   "sampling": "greedy on device"},
        "prefill": {"value": round(t / (prefill_ms / 1000), 1), "tokens": t, "ms": round(prefill_ms, 3),
                    "frac": round(prefill_tflops / PEAK_TFLOPS[args.dtype], 4),
                    **({"library_gemm_tflops": round(library, 1), "frac_of_library": round(prefill_tflops / library, 4)}
                       if library else {})},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "measured_read_ceiling": round(ceiling, 1),
                     "frac_of_measured": round(achieved / ceiling, 4)},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
