"""Command line and Python entry point, in the manner of the reference's `flow-inference`.

Commands and options keep the reference's names and meanings where it has them
(flow_engine/cli.py:48-80): `doctor`, `inspect MODEL`, `replay LOG`,
`generate MODEL --prompt ... --max-tokens N`, and the engine options
--device --dtype --max-context --kv-blocks --block-size --max-active
--prefill-chunk --target-step-ms --attention --no-prefix-cache --unfused --log.
`serve` and the draft options are not built. Added: --prompt-ids/--prompt-file
(token ids; a tokenizer is only needed for --prompt), --temperature, --seed,
--ignore-eos, --max-step-tokens, --adaptive-chunk, --no-graphs and
`random-weights CONFIG_JSON OUT --seed S` which writes a model folder.

Python: `make_engine(args) -> (Engine, tokenizer)` as in the reference
(cli.py:14-45), or `engine_for(model_folder, **options)` and `Engine.generate`.
"""
from __future__ import annotations

import argparse
from dataclasses import asdict
import json
from pathlib import Path
import platform
import sys


def _engine_options(p):
    p.add_argument("model", help="local folder with config.json and safetensors weights; nothing is downloaded")
    p.add_argument("--device", choices=["auto", "cuda"], default="auto", help="only a GPU can run this engine")
    p.add_argument("--dtype", choices=["auto", "float32", "bfloat16"], default="auto",
                   help="auto is bfloat16; float32 runs every kernel in true 32-bit")
    p.add_argument("--max-context", type=int, default=2048, help="prompt + generated tokens per request")
    p.add_argument("--kv-blocks", type=int, default=256, help="physical cache pages")
    p.add_argument("--block-size", type=int, default=16, help="tokens per page")
    p.add_argument("--max-active", type=int, default=4, help="requests admitted at once")
    p.add_argument("--prefill-chunk", type=int, default=256, help="largest prompt portion in one step")
    p.add_argument("--target-step-ms", type=float, default=50, help="step time the adaptive portion aims at")
    p.add_argument("--attention", choices=["hip"], default="hip", help="one backend: the HIP paged kernels")
    p.add_argument("--no-prefix-cache", action="store_true", help="do not reuse pages of equal prompt prefixes")
    p.add_argument("--unfused", action="store_true", help="ablation: keep q/k/v and gate/up as separate matrices")
    p.add_argument("--log", default="runs/engine.jsonl", help="JSONL event log")
    p.add_argument("--max-step-tokens", type=int, default=0, help="token budget of one step (0: max-active + prefill-chunk)")
    p.add_argument("--adaptive-chunk", action="store_true", help="size prompt portions by measured step time")
    p.add_argument("--no-graphs", action="store_true", help="never replay decode steps from HIP graphs")
    p.add_argument("--no-lookahead", action="store_true", help="read every turn's tokens before the next turn is put on the device")


def build_parser():
    from .config.registry import registered_architectures
    names = ", ".join(registered_architectures()) or "none"
    parser = argparse.ArgumentParser(prog="flow-inference",
                                     description=f"Inference engine for AMD MI355X; registered architectures: {names}")
    sub = parser.add_subparsers(dest="command", required=True)
    sub.add_parser("doctor", help="read-only report of the runtime and the accelerator")
    inspect = sub.add_parser("inspect", help="validate config.json and explain the cache allocation; no weights are read")
    inspect.add_argument("model")
    inspect.add_argument("--kv-blocks", type=int, default=256)
    inspect.add_argument("--block-size", type=int, default=16)
    replay = sub.add_parser("replay", help="print the scheduler events of a JSONL log (no inference)")
    replay.add_argument("log")
    gen = sub.add_parser("generate", help="generate tokens for one prompt")
    _engine_options(gen)
    gen.add_argument("--prompt", help="text; needs the model folder's tokenizer with a chat template")
    gen.add_argument("--prompt-ids", help="comma-separated token ids")
    gen.add_argument("--prompt-file", help="file with token ids separated by commas or white space")
    gen.add_argument("--max-tokens", type=int, default=128)
    gen.add_argument("--temperature", type=float, default=0.0)
    gen.add_argument("--seed", type=int, default=0)
    gen.add_argument("--ignore-eos", action="store_true")
    rnd = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    rnd.add_argument("config", help="a config.json (or a folder that holds one)")
    rnd.add_argument("out", help="folder to write config.json and model.safetensors into")
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--std", type=float, default=0.02)
    rnd.add_argument("--store-dtype", choices=["bfloat16", "float32"], default="bfloat16")
    return parser


def resolve_device_dtype(args):
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("no GPU is visible: this engine has no CPU path")
    dtype = "bfloat16" if args.dtype == "auto" else args.dtype
    return "cuda:0", dtype


_PROMPT_OPTIONS = ("--prompt", "--prompt-ids")


def without_prompts(argv):
    """ARGV with the value of every prompt option replaced: what a user asks never reaches a log file."""
    shown, hide_next = [], False
    for word in argv:
        name, eq, _ = word.partition("=")
        if hide_next:
            shown.append("[REDACTED]")
            hide_next = False
        elif name in _PROMPT_OPTIONS and eq:
            shown.append(name + "=[REDACTED]")
        else:
            shown.append(word)
            hide_next = word in _PROMPT_OPTIONS
    return shown


def _engine_config(args, dtype):
    from .config import EngineConfig
    return EngineConfig(
        dtype=dtype, max_context=args.max_context, kv_blocks=args.kv_blocks, block_size=args.block_size,
        max_active=args.max_active, prefix_cache=not args.no_prefix_cache,
        prefill_chunk=args.prefill_chunk, min_prefill_chunk=min(16, args.prefill_chunk),
        target_step_ms=args.target_step_ms, adaptive_chunk=args.adaptive_chunk,
        max_step_tokens=args.max_step_tokens, use_graphs=not args.no_graphs, lookahead=not args.no_lookahead)


def _chat_tokenizer(folder):
    """The model folder's own tokenizer (files only: no model code of the library runs, nothing is fetched).
    Without a chat template a text prompt is refused rather than wrapped in a guessed one (flow_engine/cli.py:40-42)."""
    from transformers import AutoTokenizer
    tokenizer = AutoTokenizer.from_pretrained(str(folder), local_files_only=True, trust_remote_code=False)
    if not tokenizer.chat_template:
        raise ValueError("a tokenizer chat_template is required; no template will be guessed")
    return tokenizer


def make_engine(args, argv=None):
    """(Engine, tokenizer or None) from parsed `generate` options (flow_engine/cli.py:14-45).

    ARGV is the command line to record in the log's first event (default: the process's own), prompts removed.
    """
    from .engine import Engine, Trace
    from .weights import load_model
    import torch

    device, dtype = resolve_device_dtype(args)
    engine_config = _engine_config(args, dtype)          # a bad option fails before any weight is read
    folder = Path(args.model).resolve(strict=True)
    trace = Trace(args.log)
    trace.emit("launch", argv=without_prompts(sys.argv if argv is None else argv), python=sys.version,
               torch=torch.__version__, device=device, dtype=dtype)
    print(f"reading weights from {folder} onto {device} as {dtype}", file=sys.stderr, flush=True)
    model = load_model(folder, dtype=dtype, device=device, packed=not args.unfused)
    tokenizer = _chat_tokenizer(folder) if getattr(args, "prompt", None) else None
    engine = Engine(model, engine_config, trace)
    trace.emit("loaded", engine=asdict(engine_config), model=model.config.describe(),
               kv_bytes=engine.cache.allocated_bytes)
    return engine, tokenizer


def engine_for(model_folder, **options):
    """An Engine for MODEL_FOLDER; OPTIONS are `generate`'s long option names with underscores."""
    argv = ["generate", str(model_folder), "--prompt-ids", "0"]
    args = build_parser().parse_args(argv)
    for key, value in options.items():
        if not hasattr(args, key):
            raise TypeError(f"unknown engine option {key!r}")
        setattr(args, key, value)
    if "log" not in options:
        args.log = None
    return make_engine(args)[0]


def _prompt_ids(args, tokenizer):
    given = [v for v in (args.prompt, args.prompt_ids, args.prompt_file) if v]
    if len(given) != 1:
        raise SystemExit("give exactly one of --prompt, --prompt-ids, --prompt-file")
    if args.prompt:
        return list(tokenizer.apply_chat_template([{"role": "user", "content": args.prompt}], tokenize=True,
                                                  add_generation_prompt=True))
    text = args.prompt_ids if args.prompt_ids else Path(args.prompt_file).read_text()
    return [int(v) for v in text.replace(",", " ").split()]


def main(argv=None):
    parser = build_parser()
    args = parser.parse_args(argv)
    if args.command == "doctor":
        import torch
        report = {"python": sys.version, "platform": platform.platform(), "torch": torch.__version__,
                  "hip": getattr(torch.version, "hip", None), "gpu": torch.cuda.is_available()}
        if torch.cuda.is_available():
            props = torch.cuda.get_device_properties(0)
            report.update(device=props.name, arch=getattr(props, "gcnArchName", None),
                          memory_bytes=props.total_memory, compute_units=props.multi_processor_count)
        from .kernels import build
        report["kernel_library"] = str(build.find_library() or "not built yet")
        print(json.dumps(report, indent=2))
    elif args.command == "inspect":
        from .config import build_model, read_model_config
        if min(args.kv_blocks, args.block_size) < 1:
            parser.error("positive block count and size are required")
        c = read_model_config(args.model)
        layout = build_model(c).cache_layout()
        tokens = args.kv_blocks * args.block_size
        # Two figures where they differ: the reference's formula over the checkpoint's head size, and what the
        # device holds (the kernels lay a head out in multiples of 16 elements, the tail zeros).
        formula = {f"kv_{name}_bytes_by_formula": c.kv_bytes_per_token(size) * tokens
                   for name, size in (("bf16", 2), ("fp32", 4)) if hasattr(c, "kv_bytes_per_token")
                   and c.kv_bytes_per_token(size) != layout.bytes_per_token(size)}
        print(json.dumps({"architecture": c.describe(),
                          "kv_formula": "2 * layers * KV_heads * head_dim * bytes_per_element * blocks * block_size"
                                        + (" (on the device head_dim is rounded up to a multiple of 16)" if formula else ""),
                          "kv_bf16_bytes": layout.bytes_per_token(2) * tokens,
                          "kv_fp32_bytes": layout.bytes_per_token(4) * tokens,
                          **formula,
                          "cache_groups": [{"layers": len(g.slots), "kv_heads": g.spec.kv_heads,
                                            "head_dim": g.spec.head_dim, "window": g.spec.window}
                                           for g in layout.groups],
                          "excludes": ["weights", "activations and scratch buffers", "runtime/allocator"]}, indent=2))
    elif args.command == "replay":
        from .engine.trace import read_events
        for event in read_events(args.log):
            print(json.dumps(event, ensure_ascii=False))
    elif args.command == "random-weights":
        from .config import config_from_dict
        from .weights import write_model_folder
        src = Path(args.config)
        src = src / "config.json" if src.is_dir() else src
        config = config_from_dict(json.loads(src.read_text()))
        out = write_model_folder(args.out, config, args.seed, args.std, args.store_dtype)
        print(str(out))
    else:
        _generate(args, ["flow-inference", *argv] if argv is not None else None)
    return 0


def _generate(args, argv):
    """`generate`: one request through the engine's worker thread; the tokens (or their text) on standard
    output, the terminal event with its usage counts on standard error (flow_engine/cli.py:107-118)."""
    engine, tokenizer = make_engine(args, argv)
    try:
        request = engine.submit(_prompt_ids(args, tokenizer), args.max_tokens, temperature=args.temperature,
                                seed=args.seed, ignore_eos=args.ignore_eos)
        engine.start()
        verdict = next(event for event in iter(request.events.get, None) if event["type"] == "done")
        if verdict["error"]:
            raise RuntimeError(verdict["error"])
        generated = request.output
        print(tokenizer.decode(generated, skip_special_tokens=True) if tokenizer is not None
              else " ".join(map(str, generated)))
        print(json.dumps(verdict), file=sys.stderr)
    finally:
        engine.close()


if __name__ == "__main__":
    sys.exit(main())
