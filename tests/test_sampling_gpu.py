"""The temperature sampler at real vocabulary sizes, and the engine's sampled tokens, against an inverse CDF
that is computed here in float64 from the same uniform numbers (flow_engine/engine.py:157: the probabilities
are softmax(logits / T); the engine draws by inverse CDF over the words in index order, the uniform number of
a draw being a function of (the request's seed, the index of the output token)).

A drawn id is right iff u * total lies inside that word's own interval of the cumulative sum. The intervals
are widened only by what float32 summation can be off by, and the logits are made wide enough that nearly every
interval is many times wider than that: the tests cannot pass by tolerance.
"""
import pytest
import torch

import plain_model as plain
from tiny_configs import make_folder

pytestmark = pytest.mark.gpu

#: what a float32 sum of up to 152,064 exponentials (pieces of a thread, 256 pieces, 64 chunks, each added in
#: order) and the float32 exponentials themselves may be off by, relative to the total: a few hundred additions
#: in a row, each good to 6e-8 of the running sum (measured: the furthest draw lay 7e-8 outside its exact interval)
SUM_SLACK = 2e-6


@pytest.fixture(scope="module")
def ops(device):
    from tessweave_engine_amd.kernels import ops as o
    return o


def check_draws(ops, logits, temps, seeds, counters, ids):
    """Every ids[r] against the float64 inverse CDF of row r. Returns how many rows were SHARP: the target lies
    further than ten times the slack from both edges of the drawn word's interval, so no other id passes."""
    rows = logits.shape[0]
    sharp, outside = 0, 0.0
    for r in range(rows):
        t = float(torch.tensor(temps[r], dtype=torch.float32))
        x = logits[r].double()
        weights = torch.exp((x - x.max()) / t)
        cdf = torch.cumsum(weights, 0)
        total = float(cdf[-1])
        target = float(ops.sampling_uniform(seeds[r], counters[r])) * total
        i = int(ids[r])
        assert 0 <= i < logits.shape[1]
        below = float(cdf[i - 1]) if i else 0.0
        above = float(cdf[i])
        slack = SUM_SLACK * total
        assert below - slack <= target <= above + slack, (
            f"row {r} (T {t}, seed {seeds[r]}, token {counters[r]}): drew word {i}, whose interval is "
            f"[{below / total:.9f}, {above / total:.9f}] of the total; the target is {target / total:.9f}, which "
            f"belongs to word {int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))}")
        assert float(weights[i]) > 0.0
        outside = max(outside, (below - target) / total, (target - above) / total)
        if target - below > 10 * slack and above - target > 10 * slack:
            sharp += 1
    print(f"{rows} draws over {logits.shape[1]} words: {sharp} well inside their interval; the furthest outside its exact "
          f"interval by {max(outside, 0.0):.2e} of the total")
    return sharp


@pytest.mark.parametrize("vocab", [152064, 389, 63 * 64 + 1])
@pytest.mark.parametrize("temperature", [0.3, 0.8, 2.0])
def test_sampled_ids_against_a_float64_inverse_cdf(ops, device, vocab, temperature):
    """Random logits whose spread grows with T (so that the words that get drawn keep intervals far wider than
    float32's summation error), seeds and token indices all different, T per row; the vocabulary of the 7B
    models (2,376 words a chunk, 10 a thread), a small odd one (its last chunks are empty), and one that leaves a
    single word for the last chunk."""
    rows = 200
    g = torch.Generator().manual_seed(int(temperature * 10) + vocab)
    logits = (torch.randn(rows, vocab, generator=g) * (4.0 * temperature)).to(device)
    temps = [temperature] * rows
    seeds = [1000003 * r + 17 for r in range(rows)]
    counters = [(r * 7) % 50 for r in range(rows)]
    ids = torch.full((rows,), -1, dtype=torch.int32, device=device)
    ops.sample_rows(logits, ids, temperature=torch.tensor(temps, device=device),
                    seeds=torch.tensor(seeds, dtype=torch.int64, device=device),
                    counters=torch.tensor(counters, dtype=torch.int32, device=device))
    sharp = check_draws(ops, logits, temps, seeds, counters, ids.cpu())
    assert sharp >= 0.7 * rows, f"only {sharp} of {rows} draws fell well inside their word's interval"
    assert len(set(ids.tolist())) > rows // 4                   # many different words were drawn


@pytest.mark.parametrize("vocab", [152064, 5000])
def test_draws_land_on_the_right_side_of_every_edge_of_the_scan(ops, device, vocab):
    """Equal weights on words that sit on the edges of the sampler's own cuts (the first and last word of a
    vocabulary chunk and of a thread's piece of a chunk, the first and last word of all), nothing elsewhere:
    the cumulative sum is a staircase of equal steps, a draw that hands the running sum wrongly from chunk to
    piece or from piece to word lands on a neighbouring step, and every step is some 4 % of the total wide."""
    chunks, threads = 64, 256
    width = -(-vocab // chunks)
    piece = -(-width // threads)
    edges = {0, vocab - 1}
    for c in (1, 2, 31, 63):
        begin = c * width
        edges |= {begin - 1, begin, begin + piece - 1, begin + piece, begin + 2 * piece - 1, min(vocab - 1, begin + width - 1)}
    edges = sorted(e for e in edges if 0 <= e < vocab)
    rows = 300
    logits = torch.full((rows, vocab), -80.0)
    logits[:, edges] = 3.0
    logits = logits.to(device)
    temps = [0.7] * rows
    seeds = [77 + r for r in range(rows)]
    counters = [r % 3 for r in range(rows)]
    ids = torch.full((rows,), -1, dtype=torch.int32, device=device)
    ops.sample_rows(logits, ids, temperature=torch.tensor(temps, device=device),
                    seeds=torch.tensor(seeds, dtype=torch.int64, device=device),
                    counters=torch.tensor(counters, dtype=torch.int32, device=device))
    got = ids.cpu()
    assert set(got.tolist()) <= set(edges)
    sharp = check_draws(ops, logits, temps, seeds, counters, got)
    assert sharp >= 0.95 * rows
    assert len(set(got.tolist())) >= len(edges) - 2              # (300 draws over some 25 steps: nearly every step is met)


# ---- the engine's sampled tokens against the plain implementation's logits -------------------------------------
def test_the_engines_sampled_tokens_are_the_inverse_cdf_draws_over_the_plain_logits(ops, tmp_path, device):
    """The second tiny configuration's workload in 32-bit: five requests of 1 to 100 prompt tokens arriving
    staggered, prompt portions of 13 beside decode tokens, temperature 0.8 (and 1.4, and one greedy request),
    24 tokens each. Token n of a request must be the word whose interval of the cumulative softmax(plain logits /
    T) holds the uniform number of (seed, n); a draw within 1e-5 of an edge is not compared (the engine's logits
    differ from the plain ones by float32 rounding), and there must be few of those."""
    from tessweave_engine_amd.cli import engine_for
    cfg, page = make_folder(tmp_path, "B")
    config, weights = plain.read_folder(tmp_path)
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (1, 9, 40, 64, 100)]
    temps = [0.8, 0.8, 1.4, 0.0, 0.8]
    seeds = [11, 2 ** 40 + 5, 13, 14, 2 ** 62 + 1]
    count = 24
    for lookahead in (True, False):
        e = engine_for(tmp_path, dtype="float32", block_size=page, kv_blocks=128, max_context=256, prefill_chunk=13,
                       max_active=4, no_prefix_cache=True, no_lookahead=not lookahead)
        requests = []
        for p, t, s in zip(prompts, temps, seeds):
            requests.append(e.submit(p, count, temperature=t, seed=s, ignore_eos=True))
            e.step()                                             # arrivals are staggered: one turn apart
            e.step()
        e.drain()
        e.close()
        compared = skipped = 0
        for r, p, t, s in zip(requests, prompts, temps, seeds):
            assert len(r.output) == count
            logits = plain.forward(config, weights, p + r.output[:-1])[len(p) - 1:]      # row n decides output token n
            for n, token in enumerate(r.output):
                if t == 0.0:
                    assert token == int(logits[n].argmax())
                    compared += 1
                    continue
                probs = plain.softmax_temperature(logits[n].double(), t).double()
                cdf = torch.cumsum(probs, 0)
                target = float(ops.sampling_uniform(s, n)) * float(cdf[-1])
                want = int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))
                below = float(cdf[want - 1]) if want else 0.0
                if min(target - below, float(cdf[want]) - target) < 1e-5:
                    skipped += 1
                    continue
                assert token == want, (lookahead, p[:3], n, token, want)
                compared += 1
        assert compared >= 5 * count - 6, (compared, skipped)
