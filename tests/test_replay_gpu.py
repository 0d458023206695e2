"""Trace replay against the plain implementation: whole, last 32 one by one, changing portions, mixed.

Every logits row the engine returns is compared with the plain implementation's
row for the same (request, position). float32 bar: the two sides sum in
different orders (MFMA tiles on the GPU, library routines on the CPU), so a few
float32 roundings of O(1) logits are allowed: atol 5e-6, rtol 2e-5 (the
reference's own bar between two CPU paths is atol 2e-6, rtol 2e-5,
tests/test_engine.py:65). bfloat16 bar: 2 % of the largest logit, absolute.
"""
import io
import json
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_model as plain
from tiny_configs import TINY, make_folder

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent

LENGTHS = {"A": [37, 49, 70, 33, 64, 40], "B": [33, 41, 64, 100, 124, 35, 50], "C": [36, 65, 97, 130, 34, 48],
           "B320": [33, 41, 64, 100, 124, 35, 50]}


def round64(n):
    return (n + 63) // 64 * 64


@pytest.fixture(scope="module", params=["A", "B", "C", "B320"])
def tiny(request, tmp_path_factory, device):
    name = request.param
    folder = tmp_path_factory.mktemp(f"tiny{name}")
    cfg, page = make_folder(folder, name)
    config, weights = plain.read_folder(folder)
    g = torch.Generator().manual_seed(100 + len(name) + ord(name[0]))
    requests = {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()
                for i, n in enumerate(LENGTHS[name])}
    want = {rid: plain.forward(config, weights, toks).numpy() for rid, toks in requests.items()}
    return dict(name=name, folder=folder, page=page, cfg=cfg, requests=requests, want=want)


def run_trace(tiny, dtype, steps, max_tokens, out_dir, extra=()):
    from tessweave_engine_amd.engine import replay
    args = replay.parse_args(["--model", str(tiny["folder"]), "--dtype", dtype, "--out", str(out_dir),
                              "--max-tokens", str(max_tokens), "--page-size", str(tiny["page"]), *extra])
    sink = io.StringIO()
    replay.run(args, [json.dumps(s) for s in steps], out=sink)
    assert sink.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    vocab = tiny["cfg"]["vocab_size"]
    got = {}
    for s in steps:
        path = Path(out_dir) / f"{s['step']}.f32"
        wanted = sum(len(e["want"]) for e in s["entries"])
        assert path.exists() == (wanted > 0)
        if wanted:
            got[s["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
    return got


def compare(tiny, dtype, steps, got, starts):
    """STARTS[(step, request id)] = position of the entry's first token.

    A model that also brings "exact" (the plain implementation's logits in float64) gets a calibrated float32
    bar instead of the fixed one: the absolute part is four times what the plain implementation in float32
    ("want") is off from float64 at worst, plus 1e-6; the relative part is the reference's own 2e-5
    (tests/test_engine.py:65). Sums over a few thousand terms round differently in every order; how much
    depends on the widths, which random configurations vary a hundredfold, and a tied head gives a token's
    own logit a size of tens, where a chain of 32-bit additions is off by several units in the last place.
    """
    if dtype == "float32" and "exact" in tiny:
        rows = []
        for s in steps:
            row = 0
            for e in s["entries"]:
                base = starts[(s["step"], e["id"])]
                for w in e["want"]:
                    rows.append((e["id"], base + w, s["step"], got[s["step"]][row]))
                    row += 1
        worst_plain = max(float(np.abs(tiny["want"][rid][pos] - tiny["exact"][rid][pos]).max()) for rid, pos, _, _ in rows)
        atol = 4 * worst_plain + 1e-6
        worst_engine = 0.0
        for rid, pos, step, have in rows:
            exact = tiny["exact"][rid][pos]
            err = np.abs(have - exact)
            worst_engine = max(worst_engine, float(err.max()))
            assert (err <= atol + 2e-5 * np.abs(exact)).all(), (
                f"{tiny['name']} float32: request {rid} position {pos} (step {step}): off from float64 by "
                f"{err.max():.3e}; plain float32 is off by at most {worst_plain:.3e}, largest logit {np.abs(exact).max():.3f}")
        return worst_engine
    worst = 0.0
    for s in steps:
        row = 0
        for e in s["entries"]:
            base = starts[(s["step"], e["id"])]
            for w in e["want"]:
                want = tiny["want"][e["id"]][base + w]
                have = got[s["step"]][row]
                row += 1
                if dtype == "float32":
                    ok = np.allclose(have, want, atol=5e-6, rtol=2e-5)
                else:
                    ok = np.abs(have - want).max() <= 0.02 * np.abs(want).max()
                worst = max(worst, float(np.abs(have - want).max()))
                assert ok, (f"{tiny['name']} {dtype}: request {e['id']} position {base + w} (step {s['step']}): "
                            f"max abs error {np.abs(have - want).max():.3e}, largest logit {np.abs(want).max():.3f}")
    return worst


def sequential(tiny, cut):
    """One request after the other; CUT(tokens) gives the sizes of its steps."""
    steps, starts, n = [], {}, 0
    for rid, toks in tiny["requests"].items():
        sizes = cut(len(toks))
        assert sum(sizes) == len(toks)
        pos = 0
        for i, size in enumerate(sizes):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[pos:pos + size], "want": list(range(size))}],
                          "end": [rid] if i == len(sizes) - 1 else []})
            starts[(n, rid)] = pos
            pos += size
            n += 1
    return steps, starts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole(tiny, dtype, tmp_path):
    steps, starts = sequential(tiny, lambda t: [t])
    biggest = max(round64(len(t)) for t in tiny["requests"].values())
    got = run_trace(tiny, dtype, steps, biggest, tmp_path)
    compare(tiny, dtype, steps, got, starts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [True, False])
def test_last_32_one_by_one(tiny, dtype, graphs, tmp_path):
    steps, starts = sequential(tiny, lambda t: ([t - 32] if t > 32 else []) + [1] * min(t, 32))
    biggest = max(round64(len(t)) for t in tiny["requests"].values())
    got = run_trace(tiny, dtype, steps, biggest, tmp_path, extra=() if graphs else ("--no-graphs",))
    compare(tiny, dtype, steps, got, starts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(tiny, dtype, tmp_path):
    pattern = [7, 13, 5, 3, 2, 2, 11, 2, 17, 4, 2, 9]

    def cut(t):
        sizes, i = [], 0
        while t:
            size = min(pattern[i % len(pattern)], t)
            if t - size == 1:          # never leave a single token: every portion has at least two
                size += 1
            sizes.append(size)
            t -= size
            i += 1
        return sizes
    steps, starts = sequential(tiny, cut)
    assert min(len(s["entries"][0]["tokens"]) for s in steps) == 2
    biggest = max(round64(len(t)) for t in tiny["requests"].values())
    got = run_trace(tiny, dtype, steps, biggest, tmp_path)
    compare(tiny, dtype, steps, got, starts)


def mixed_trace(tiny, seed):
    """Up to four live requests; prompt portions beside single tokens; requests skip steps; arrivals staggered."""
    rng = random.Random(seed)
    pending = list(tiny["requests"].items())
    live, steps, starts, n, peak = {}, [], {}, 0, 0
    while pending or live:
        while pending and len(live) < 4 and (not live or rng.random() < 0.5):
            rid, toks = pending.pop(0)
            live[rid] = dict(tokens=toks, pos=0, prompt=rng.randrange(2, len(toks) - 1))
        peak = max(peak, sum(round64(len(r["tokens"])) for r in live.values()))
        entries, ended = [], []
        for rid, r in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                    # left out of this step, goes on later
            left = len(r["tokens"]) - r["pos"]
            if r["pos"] < r["prompt"]:
                size = min(rng.choice([2, 3, 5, 7, 13]), r["prompt"] - r["pos"])
                if r["prompt"] - r["pos"] - size == 1:
                    size += 1
            else:
                size = 1
            size = min(size, left)
            want = list(range(size)) if rng.random() < 0.8 else []
            entries.append({"id": rid, "tokens": r["tokens"][r["pos"]:r["pos"] + size], "want": want})
            starts[(n, rid)] = r["pos"]
            r["pos"] += size
            if r["pos"] == len(r["tokens"]):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": n, "entries": entries, "end": ended})
            n += 1
    return steps, starts, peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [0, 1])
def test_mixed_with_few_pages(tiny, dtype, seed, tmp_path):
    steps, starts, peak = mixed_trace(tiny, seed)
    assert max(len(s["entries"]) for s in steps) >= 3
    assert any(len(e["tokens"]) > 1 for s in steps for e in s["entries"] if any(len(o["tokens"]) == 1 for o in s["entries"]))
    total = sum(round64(len(t)) for t in tiny["requests"].values())
    assert peak < total                                       # the pool is smaller than all requests: pages are reused
    got = run_trace(tiny, dtype, steps, peak, tmp_path)
    compare(tiny, dtype, steps, got, starts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page", [12, 24, 48, 20])
def test_pages_whose_size_is_no_power_of_two(tiny, dtype, page, tmp_path):
    """Every multiple of 4 is a page size the engine takes; the fast bfloat16 attention kernels want powers of
    two, so these run the kernels that divide by the page size: mixed with few pages, and the last 32 one by one."""
    other = dict(tiny, page=page)
    steps, starts, peak = mixed_trace(other, 3)
    got = run_trace(other, dtype, steps, peak, tmp_path / "mixed")
    compare(other, dtype, steps, got, starts)
    steps, starts = sequential(other, lambda t: ([t - 32] if t > 32 else []) + [1] * min(t, 32))
    biggest = max(round64(len(t)) for t in other["requests"].values())
    got = run_trace(other, dtype, steps, biggest, tmp_path / "single")
    compare(other, dtype, steps, got, starts)


def test_ways_of_cutting_agree_beyond_rounding(tiny, tmp_path):
    """float32: whole, one-by-one and mixed replays give the same logits up to summation order."""
    whole, s0 = sequential(tiny, lambda t: [t])
    single, s1 = sequential(tiny, lambda t: [1] * t)
    biggest = max(round64(len(t)) for t in tiny["requests"].values())
    a = run_trace(tiny, "float32", whole, biggest, tmp_path / "a")
    b = run_trace(tiny, "float32", single, biggest, tmp_path / "b")
    rows_a = np.concatenate([a[s["step"]] for s in whole])
    rows_b = np.concatenate([b[s["step"]] for s in single])
    assert np.abs(rows_a - rows_b).max() < 5e-6


def test_program_as_a_user_runs_it(tiny, tmp_path):
    """bin/trace_run as a separate process: options, stdin protocol, files, exit code."""
    rid, toks = next(iter(tiny["requests"].items()))
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": rid, "tokens": toks[20:22], "want": []}], "end": []},
             {"step": 5, "entries": [{"id": rid, "tokens": toks[22:23], "want": [0]}], "end": [rid]}]
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(tiny["folder"]),
                           "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64",
                           "--page-size", str(tiny["page"])],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == ["done", "0", "done", "1", "done", "5"]
    vocab = tiny["cfg"]["vocab_size"]
    first = np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, vocab)
    last = np.fromfile(tmp_path / "o" / "5.f32", dtype="<f4").reshape(1, vocab)
    assert not (tmp_path / "o" / "1.f32").exists()
    want = tiny["want"][rid]
    np.testing.assert_allclose(first, want[[0, 19]], atol=5e-6, rtol=2e-5)
    np.testing.assert_allclose(last, want[[22]], atol=5e-6, rtol=2e-5)
    # more tokens than the pool was made for is an error, not a wrong result
    too_many = [{"step": 0, "entries": [{"id": "x", "tokens": (toks * 4)[:129], "want": []}], "end": []}]
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(tiny["folder"]),
                           "--dtype", "float32", "--out", str(tmp_path / "p"), "--max-tokens", "128",
                           "--page-size", str(tiny["page"])],
                          input=json.dumps(too_many[0]) + "\n", capture_output=True, text=True, timeout=110)
    assert proc.returncode != 0 and "done" not in proc.stdout
