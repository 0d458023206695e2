"""The float32 correctness run at the Qwen2.5-7B shape (the reference's method: tools/validate_model.py:87-95,
chunked logits against whole-sequence logits in 32-bit).

4 of the 28 layers, at full width (hidden 3,584, 28 query heads over 4 key/value heads of 128, feed-forward
18,944) and with the full vocabulary of 152,064 (an untied head): the head's 152,064 columns and the growth of
the error over several wide layers are what a one-layer, small-vocabulary model does not show. All of it through
trace replay, in ONE session whose pool is sized for the mixed part, so that pages are used again:

  whole       every request in one step
  last 32     most of a request in one step, its last 32 tokens one by one (from HIP graphs)
  portions    a request in portions of changing size, down to two tokens
  mixed       up to four live requests, portions beside single tokens, few pages

The weights are drawn on the GPU (two billion values) and the plain implementation runs there too, in float64
(the yardstick), in float32 and in bfloat16. Both bars are calibrated rather than fixed, because rounding errors
grow with depth, width and the number of columns the largest error is taken over (with one wide layer and 4,099
columns bfloat16 is off by 1 % of the largest logit, with four layers and 152,064 columns by 2 %: the square
root of the depth). float32: the engine may be off from float64 by at most twice what the plain
implementation in float32 is off (+ 1e-6). bfloat16: the engine, which keeps the residual stream, the softmax
and every sum in 32-bit, must be closer to float64 than the plain implementation with every tensor and every
intermediate result in bfloat16 is.
"""
import io
import json
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_model as plain
import test_replay_gpu as replay_tests

pytestmark = pytest.mark.gpu

LAYERS, LAYERS_OF = 4, 28
SHAPE = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=LAYERS, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
    intermediate_size=18944, vocab_size=152064, rope_theta=1e6, rms_norm_eps=1e-6,
    tie_word_embeddings=False, use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu")
LENGTHS = {"a": 200, "b": 70, "c": 131, "d": 40, "e": 97, "f": 52}
PAGE = 16


@pytest.fixture(scope="module")
def shape7b(tmp_path_factory, device):
    from tessweave_engine_amd.config import config_from_dict
    from tessweave_engine_amd.weights import write_model_folder
    folder = tmp_path_factory.mktemp("qwen7b_shape")
    write_model_folder(folder, config_from_dict(SHAPE), 2025, device=device)
    g = torch.Generator().manual_seed(7)
    requests = {rid: torch.randint(0, SHAPE["vocab_size"], (n,), generator=g).tolist() for rid, n in LENGTHS.items()}
    exact, single, half = {}, {}, {}
    for dtype, store in ((torch.float64, exact), (torch.float32, single), (torch.bfloat16, half)):
        config, w = plain.read_folder(folder, dtype, device)
        with torch.device(device):
            for rid, toks in requests.items():
                store[rid] = plain.forward(config, w, toks).cpu().numpy()     # float32 [T, vocab]; float64 was summed in 64-bit
        del w
        torch.cuda.empty_cache()
    yield dict(folder=folder, requests=requests, exact=exact, single=single, half=half)
    for f in Path(folder).iterdir():
        f.unlink()


def session(requests):
    """One trace with the four ways of cutting, each under request ids of its own.
    Returns (steps, {(step, id): (request, first position)}, most tokens live at once)."""
    steps, origin = [], {}
    peak = 0

    def add(entries, end, live_tokens):
        nonlocal peak
        n = len(steps)
        steps.append({"step": n, "entries": [{"id": i, "tokens": t, "want": w} for i, _, _, t, w in entries], "end": end})
        for i, rid, first, _, _ in entries:
            origin[n, i] = (rid, first)
        peak = max(peak, live_tokens)

    # whole
    for rid, toks in requests.items():
        add([(f"w.{rid}", rid, 0, toks, list(range(len(toks))))], [f"w.{rid}"], replay_tests.round64(len(toks)))
    # most of request a in one step, its last 32 tokens one by one
    toks = requests["a"]
    head = len(toks) - 32
    add([("l.a", "a", 0, toks[:head], [head - 1])], [], 256)
    for i in range(32):
        add([("l.a", "a", head + i, [toks[head + i]], [0])], ["l.a"] if i == 31 else [], 256)
    # request c in portions of changing size, down to two tokens
    toks, pos = requests["c"], 0
    pattern = [7, 13, 5, 3, 2, 2, 11, 2, 17, 4, 2, 9, 33, 2, 6]
    i = 0
    while pos < len(toks):
        size = min(pattern[i % len(pattern)], len(toks) - pos)
        if len(toks) - pos - size == 1:
            size += 1
        last = pos + size == len(toks)
        add([("p.c", "c", pos, toks[pos:pos + size], list(range(size)))], ["p.c"] if last else [], 192)
        pos += size
        i += 1
    # mixed: the generator of the tiny replays, under ids of its own
    mixed, starts, mixed_peak = replay_tests.mixed_trace(dict(requests={f"m.{r}": t for r, t in requests.items()}), 4)
    for s in mixed:
        add([(e["id"], e["id"][2:], starts[s["step"], e["id"]], e["tokens"], e["want"]) for e in s["entries"]],
            s["end"], mixed_peak)
    return steps, origin, peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_full_width_layers_and_the_full_vocabulary_through_replay(shape7b, dtype, tmp_path):
    from tessweave_engine_amd.engine import replay
    steps, origin, peak = session(shape7b["requests"])
    total = sum(replay_tests.round64(n) for n in LENGTHS.values())
    assert peak < total                                   # fewer pages than all requests need: pages are used again
    assert any(len(s["entries"]) >= 3 for s in steps) and min(len(e["tokens"]) for s in steps for e in s["entries"]) == 1
    args = replay.parse_args(["--model", str(shape7b["folder"]), "--dtype", dtype, "--out", str(tmp_path),
                              "--max-tokens", str(peak), "--page-size", str(PAGE)])
    sink = io.StringIO()
    replay.run(args, [json.dumps(s) for s in steps], out=sink)
    vocab = SHAPE["vocab_size"]
    worst_engine = worst_plain = largest = 0.0
    compared = 0
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        if not wanted:
            continue
        path = Path(tmp_path) / f"{s['step']}.f32"
        got = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        path.unlink()
        row = 0
        for e in s["entries"]:
            rid, first = origin[s["step"], e["id"]]
            for w in e["want"]:
                exact = shape7b["exact"][rid][first + w]
                err = float(np.abs(got[row] - exact).max())
                top = float(np.abs(exact).max())
                worst_engine = max(worst_engine, err)
                yardstick = shape7b["single" if dtype == "float32" else "half"][rid][first + w]
                plain_err = float(np.abs(yardstick - exact).max())
                worst_plain = max(worst_plain, plain_err)
                if dtype == "bfloat16":
                    assert err <= 0.04 * top, (e["id"], first + w, s["step"], err, top)     # never grossly off
                largest = max(largest, top)
                row += 1
                compared += 1
    print(f"Qwen2.5-7B shape, {LAYERS} of {LAYERS_OF} layers, vocabulary {vocab}, {dtype}: {compared} logit rows in "
          f"{len(steps)} steps; engine off by {worst_engine:.3e}, plain {dtype} off by {worst_plain:.3e}, "
          f"largest logit {largest:.3f}")
    if dtype == "float32":
        assert worst_engine <= 2 * worst_plain + 1e-6, (worst_engine, worst_plain)
    else:
        assert worst_engine <= worst_plain, (worst_engine, worst_plain)
