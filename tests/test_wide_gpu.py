"""One decoder layer at the width of real checkpoints, through trace replay, against the plain implementation.

The tiny configurations run the kernels' small paths; this one has the sizes the
serving kernels are tuned for (hidden 3,584, 28 query heads over 4 key/value heads
of 128, feed-forward 18,944: the Qwen2.5-7B layer), so a prompt portion goes
through the large matrix tiles with split K, a decode token through the streaming
kernels with their K ranges, and attention through the head-128 instantiations.
One layer and a small odd vocabulary keep the plain implementation quick.

float32 bar: at this width the order of summation matters more than in the tiny
models (rows of 18,944 products), so the bar is calibrated instead of fixed: the
engine may differ from the plain implementation in float64 by at most four times
what the plain implementation in float32 differs from it (plus 1e-6). bfloat16
bar: 2 % of the largest logit, as in the other replay tests.
"""
import io
import json
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_model as plain

pytestmark = pytest.mark.gpu

WIDE = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=1, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
    intermediate_size=18944, vocab_size=4099, rope_theta=1e6, rms_norm_eps=1e-6,
    tie_word_embeddings=False, use_sliding_window=False, max_position_embeddings=2048, hidden_act="silu")
WIDE_SEED, WIDE_PAGE = 7, 16
LENGTHS = {"long": 330, "short": 70}


@pytest.fixture(scope="module")
def wide(tmp_path_factory, device):
    from tessweave_engine_amd.config import config_from_dict
    from tessweave_engine_amd.weights import write_model_folder
    folder = tmp_path_factory.mktemp("wide")
    write_model_folder(folder, config_from_dict(WIDE), WIDE_SEED)
    g = torch.Generator().manual_seed(77)
    requests = {rid: torch.randint(0, WIDE["vocab_size"], (n,), generator=g).tolist() for rid, n in LENGTHS.items()}
    config, w64 = plain.read_folder(folder, torch.float64)
    exact = {rid: plain.forward(config, w64, toks).numpy() for rid, toks in requests.items()}
    del w64
    config, w32 = plain.read_folder(folder, torch.float32)
    single = {rid: plain.forward(config, w32, toks).numpy() for rid, toks in requests.items()}
    return dict(folder=folder, requests=requests, exact=exact, single=single)


def trace(requests):
    """The long request: 298 tokens in one step, then its last 32 one by one; beside them the short
    request in portions of 35, 33 and 2. Returns (steps, {(step, id): first position})."""
    long_, short = requests["long"], requests["short"]
    steps, starts = [], {}
    head = len(long_) - 32
    steps.append({"step": 0, "entries": [{"id": "long", "tokens": long_[:head], "want": list(range(head))}], "end": []})
    starts[(0, "long")] = 0
    cuts = {3: (0, 35), 9: (35, 68), 20: (68, 70)}
    for i in range(32):
        n = i + 1
        entries = [{"id": "long", "tokens": [long_[head + i]], "want": [0]}]
        starts[(n, "long")] = head + i
        if n in cuts:
            a, b = cuts[n]
            entries.append({"id": "short", "tokens": short[a:b], "want": list(range(b - a))})
            starts[(n, "short")] = a
        steps.append({"step": n, "entries": entries, "end": (["long"] if i == 31 else []) + (["short"] if n == 20 else [])})
    return steps, starts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_wide_layer_whole_decoded_and_mixed(wide, dtype, tmp_path):
    from tessweave_engine_amd.engine import replay
    steps, starts = trace(wide["requests"])
    args = replay.parse_args(["--model", str(wide["folder"]), "--dtype", dtype, "--out", str(tmp_path),
                              "--max-tokens", "512", "--page-size", str(WIDE_PAGE)])
    sink = io.StringIO()
    replay.run(args, [json.dumps(s) for s in steps], out=sink)
    vocab = WIDE["vocab_size"]
    worst_engine = worst_plain = largest = 0.0
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        got = np.fromfile(Path(tmp_path) / f"{s['step']}.f32", dtype="<f4").reshape(wanted, vocab)
        row = 0
        for e in s["entries"]:
            base = starts[(s["step"], e["id"])]
            for w in e["want"]:
                exact = wide["exact"][e["id"]][base + w]
                err = float(np.abs(got[row] - exact).max())
                if dtype == "bfloat16":
                    assert err <= 0.02 * np.abs(exact).max(), (e["id"], base + w, s["step"], err)
                worst_engine = max(worst_engine, err)
                worst_plain = max(worst_plain, float(np.abs(wide["single"][e["id"]][base + w] - exact).max()))
                largest = max(largest, float(np.abs(exact).max()))
                row += 1
    print(f"wide layer {dtype}: engine off by {worst_engine:.3e}, plain float32 off by {worst_plain:.3e}, "
          f"largest logit {largest:.3f}")
    if dtype == "float32":
        assert worst_engine <= 4 * worst_plain + 1e-6, (worst_engine, worst_plain)
