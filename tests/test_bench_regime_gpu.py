"""The sizes the benchmark times, against the plain implementation.

The other GPU tests stop at a few hundred keys and four requests. What `bench.py` measures runs elsewhere
in the same kernels: decode attention over thousands of keys cut into as many ranges as the launcher itself
chooses (most of them empty for a short request in a batch sized for long ones), decode batches of 33-64
rows (the widest instantiation of the streaming matrix kernel), graphs captured for an engine that is
opened for thousands of tokens, and a 2,048-token prompt portion through the largest matrix tiles and the
128-row attention tiles in one step. Each is compared here with the plain implementation, in both precisions.
"""
import math

import pytest
import torch

import plain_model as plain
from test_kernels_gpu import ATTN_TOL, build_paged
from tiny_configs import make_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(device):
    from tessweave_engine_amd.kernels import ops as o
    return o


def decode_case(ops, device, dtype, heads, kv_heads, d, page, lengths, k, v, q, splits_list, window=0):
    n_seqs = len(lengths)
    pages_total = sum(math.ceil(n / page) for n in lengths) + 3
    keys, values, table = build_paged(k, v, lengths, page, pages_total, device, dtype, seed=len(lengths))
    want = torch.stack([plain.attention(q[i:i + 1].float(), k[i], v[i], torch.tensor([lengths[i] - 1]),
                                        window=window or None)[0] for i in range(n_seqs)])
    qd = q.reshape(n_seqs, heads * d).to(dtype).to(device)
    q_start = torch.arange(n_seqs + 1, dtype=torch.int32, device=device)
    kv_len = torch.tensor(lengths, dtype=torch.int32, device=device)
    for splits, generic in splits_list:
        out = torch.full((n_seqs, heads * d), float("nan"), dtype=dtype, device=device)
        ws = torch.full((max(1, ops.attn_decode_workspace_floats(n_seqs, heads, d, splits)),), float("nan"), device=device)
        ops.attn_decode(qd, keys, values, table, q_start, kv_len, 0, n_seqs, out, heads, kv_heads, d, d ** -0.5,
                        window=window, splits=splits, workspace=ws, generic=generic)
        torch.testing.assert_close(out.float().cpu().reshape(n_seqs, heads, d), want, **ATTN_TOL[dtype],
                                   msg=lambda m: f"splits {splits} generic {generic}: {m}")
    return want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim", [64, 128, 256])
def test_decode_attention_with_many_key_ranges_most_of_them_empty(ops, device, dtype, head_dim):
    """16, 33 and 64 key ranges over requests of 5, 3,000, 1 and 700 keys: a short request leaves most ranges
    empty (their partial results must count for nothing), and the merge kernel runs past the ranges one pass
    of its loop takes."""
    heads, kv_heads, page = 8, 2, 16
    lengths = [5, 3000, 1, 700]
    g = torch.Generator().manual_seed(head_dim)
    k = [torch.randn(n, kv_heads, head_dim, generator=g).to(dtype).float() for n in lengths]
    v = [torch.randn(n, kv_heads, head_dim, generator=g).to(dtype).float() for n in lengths]
    q = torch.randn(len(lengths), heads, head_dim, generator=g).to(dtype)
    decode_case(ops, device, dtype, heads, kv_heads, head_dim, page, lengths, k, v, q,
                [(16, False), (33, False), (64, False), (16, True), (33, True), (64, True)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("longest,batch", [(4096, 1), (4096, 8), (32000, 1), (32000, 3)])
def test_decode_attention_at_the_benchmarks_lengths_with_the_launchers_own_ranges(ops, device, dtype, longest, batch):
    """28 query heads over 4 key/value heads of 128 (the 7B layer), 4,096 and 32,000 keys, the number of
    key ranges that the launcher picks for this batch. Every head's query points at ONE key on an edge (first,
    last, page and block edges, the edges of the chosen ranges), so a dropped or doubled key is off by O(1)
    in bfloat16 too; the other requests of the batch are short and leave most ranges empty."""
    heads, kv_heads, d, page = 28, 4, 128, 16
    splits = ops.attn_decode_splits(batch, heads, kv_heads, longest)
    assert splits > 1
    span = math.ceil(longest / splits)
    targets = [0, 1, 15, 16, 31, 32, 33, 63, 64, 255, 256, span - 1, span, span + 1, 2 * span - 1, 2 * span,
               longest // 2, longest - span - 1, longest - span, longest - 257, longest - 65, longest - 64, longest - 33,
               longest - 32, longest - 17, longest - 16, longest - 2, longest - 1]
    assert len(targets) == heads and all(0 <= t < longest for t in targets)
    lengths = [longest] + [37, 1500, 9, 2048, 1, 640, 100][:batch - 1]
    g = torch.Generator().manual_seed(longest + batch)
    unit = torch.nn.functional.normalize(torch.randn(heads, d, generator=g), dim=1)
    k = [torch.randn(n, kv_heads, d, generator=g) * 0.1 for n in lengths]
    v = [torch.randn(n, kv_heads, d, generator=g) for n in lengths]
    group = heads // kv_heads
    owner = {}
    for h, p in enumerate(targets):
        k[0][p, h // group] = unit[h] * 30.0           # several heads of a group have their own far key
        owner[p, h // group] = h                       # (two heads of a group may name the same key: the later one has it)
    k = [t.to(dtype).float() for t in k]
    v = [t.to(dtype).float() for t in v]
    q = torch.randn(len(lengths), heads, d, generator=g)
    q[0] = unit * 12.0
    q = q.to(dtype)
    want = decode_case(ops, device, dtype, heads, kv_heads, d, page, lengths, k, v, q,
                       [(splits, False), (splits, True), (1, False)])
    # the vectors do what they are for: each head of the long request returns (nearly) its target's value
    hits = 0
    for h, p in enumerate(targets):
        if owner[p, h // group] == h:
            hits += 1
            assert (want[0, h] - v[0][p, h // group]).abs().max() < 0.05, (h, p)
    assert hits >= 20


# ---- the engine opened for thousands of tokens, decode batches of 40 and 64 from graphs ----------------------------
@pytest.fixture(scope="module")
def long_model(tmp_path_factory, device):
    folder = tmp_path_factory.mktemp("longA")
    cfg, page = make_folder(folder, "A")
    cfg = dict(cfg, max_position_embeddings=8192)
    import json
    (folder / "config.json").write_text(json.dumps(cfg))
    config, weights = plain.read_folder(folder)
    return dict(folder=folder, page=page, cfg=cfg, config=config, weights=weights)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_req", [40, 64, 65, 128])
def test_decode_batches_of_40_to_128_requests_short_and_long_from_graphs(long_model, dtype, n_req):
    """An engine opened for 4,224 tokens a request: the captured decode step sizes its key ranges by the
    length class, and the batch holds requests of 3 to 4,100 tokens. Six decode steps (one eager, one captured,
    four replayed) of 40 requests (the streaming matrix kernel's 48-row form), of 64 (its 64-row form, the
    benchmark's), and of 65 and 128 (single tokens through the tiled matrix kernels, which take over above 64
    rows, where the projections also stop leaving their sums to the next kernel), every logits row against the
    plain implementation."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    page, vocab = long_model["page"], long_model["cfg"]["vocab_size"]
    n_decode, capacity = 6, 4224
    g = torch.Generator().manual_seed(48)
    prompt_lens = [4100, 1500, 3, 700] + torch.randint(1, 200, (n_req - 4,), generator=g).tolist()
    tokens = [torch.randint(0, vocab, (n + n_decode,), generator=g).tolist() for n in prompt_lens]
    want = [plain.forward(long_model["config"], long_model["weights"], t) for t in tokens]
    model = load_model(long_model["folder"], dtype=dtype, device="cuda:0")
    pages = sum(math.ceil((n + n_decode) / page) for n in prompt_lens)
    cache = CacheManager(model.cache_layout(), page, pages, n_req, dtype=dtype, device=model.device,
                         prefix_cache=False, max_request_tokens=capacity)
    stepper = Stepper(model, cache, max_step_tokens=512, max_step_seqs=n_req)
    seqs = [cache.open(f"r{i}") for i in range(n_req)]
    worst = 0.0

    def check(got, rows):
        nonlocal worst
        for r, (i, pos) in enumerate(rows):
            w = want[i][pos]
            err = float((got[r] - w).abs().max())
            worst = max(worst, err)
            if dtype == "float32":
                assert torch.allclose(got[r], w, atol=5e-6, rtol=2e-5), (i, pos, err)
            else:
                assert err <= 0.02 * float(w.abs().max()), (i, pos, err)
    # prompts: the long ones in portions of 512, the short ones several to a step
    for i in (0, 1, 3):
        for a in range(0, prompt_lens[i], 512):
            b = min(prompt_lens[i], a + 512)
            got = stepper.step([StepEntry(seqs[i], tokens[i][a:b], [b - a - 1])]).cpu()
            check(got, [(i, b - 1)])
    rest = [i for i in range(n_req) if i not in (0, 1, 3)]
    for a in range(0, len(rest), 8):
        batch = rest[a:a + 8]
        got = stepper.step([StepEntry(seqs[i], tokens[i][:prompt_lens[i]], [prompt_lens[i] - 1]) for i in batch]).cpu()
        check(got, [(i, prompt_lens[i] - 1) for i in batch])
    # decode: all of them in every step
    for s in range(n_decode):
        got = stepper.step([StepEntry(seqs[i], [tokens[i][prompt_lens[i] + s]], [0]) for i in range(n_req)]).cpu()
        check(got, [(i, prompt_lens[i] + s) for i in range(n_req)])
    assert stepper.graph_replays >= n_decode - 2
    print(f"{n_req} requests, {dtype}: worst difference {worst:.3e}")
    for seq in seqs:
        cache.close(seq)
    cache.check()
    stepper.close()


# ---- one layer at the 7B width: a 2,048-token portion in one step, then decoding past 4,096 keys ------------
WIDE = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=1, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
    intermediate_size=18944, vocab_size=1031, rope_theta=1e6, rms_norm_eps=1e-6,
    tie_word_embeddings=False, use_sliding_window=False, max_position_embeddings=8192, hidden_act="silu")


def plain_on_device(config, weights, tokens, dtype, device, rows):
    """The plain implementation's logits at ROWS, its tensors moved to the GPU (torch's float64 there) so that
    4,104 tokens through a 7B-width layer take seconds. Only the last layer's rows are cut; nothing else changes."""
    w = {k: t.to(device=device, dtype=dtype) for k, t in weights.items()}
    logits = _forward_on(config, w, tokens, device)
    return logits[rows].cpu()


def _forward_on(config, w, tokens, device):
    # plain.forward builds its index tensors on the CPU; run it under a default device instead
    with torch.device(device):
        return plain.forward(config, w, tokens)


@pytest.fixture(scope="module")
def wide_long(tmp_path_factory, device):
    from tessweave_engine_amd.config import config_from_dict
    from tessweave_engine_amd.weights import write_model_folder
    folder = tmp_path_factory.mktemp("wide_long")
    write_model_folder(folder, config_from_dict(WIDE), 11)
    g = torch.Generator().manual_seed(2048)
    n = 4096 + 8
    tokens = torch.randint(0, WIDE["vocab_size"], (n,), generator=g).tolist()
    rows = [0, 1, 127, 128, 1000, 2047, 2048, 2049, 4094, 4095] + list(range(4096, n))
    config, weights = plain.read_folder(folder, torch.float32)
    exact = plain_on_device(config, weights, tokens, torch.float64, device, rows)
    single = plain_on_device(config, weights, tokens, torch.float32, device, rows)
    return dict(folder=folder, tokens=tokens, rows=rows, exact=exact, single=single)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_2048_token_portion_in_one_step_then_decoding_past_4096_keys(wide_long, dtype):
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    tokens, rows = wide_long["tokens"], wide_long["rows"]
    model = load_model(wide_long["folder"], dtype=dtype, device="cuda:0")
    page = 16
    cache = CacheManager(model.cache_layout(), page, math.ceil(len(tokens) / page) + 1, 2, dtype=dtype,
                         device=model.device, prefix_cache=False, max_request_tokens=len(tokens) + page)
    stepper = Stepper(model, cache, max_step_tokens=2048, max_step_seqs=2)
    seq = cache.open("r")
    got = {}
    for a in (0, 2048):                                         # two portions of 2,048 tokens, each ONE step
        want_rows = [r - a for r in rows if a <= r < a + 2048]
        out = stepper.step([StepEntry(seq, tokens[a:a + 2048], want_rows)]).cpu()
        for j, r in enumerate(want_rows):
            got[r + a] = out[j].clone()
    for p in range(4096, len(tokens)):                          # then single tokens over 4,097+ keys
        got[p] = stepper.step([StepEntry(seq, [tokens[p]], [0])]).cpu()[0].clone()
    assert stepper.graph_replays >= len(tokens) - 4096 - 2
    worst_engine = worst_plain = 0.0
    for j, r in enumerate(rows):
        exact = wide_long["exact"][j].float()
        err = float((got[r] - exact).abs().max())
        worst_engine = max(worst_engine, err)
        worst_plain = max(worst_plain, float((wide_long["single"][j] - exact).abs().max()))
        if dtype == "bfloat16":
            assert err <= 0.02 * float(exact.abs().max()), (r, err)
    print(f"2,048-token portions + decode past 4,096 keys, {dtype}: engine off by {worst_engine:.3e}, "
          f"plain float32 off by {worst_plain:.3e}")
    if dtype == "float32":
        assert worst_engine <= 2 * worst_plain + 1e-6, (worst_engine, worst_plain)
    cache.close(seq)
    stepper.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_across_a_length_class_takes_a_second_graph_and_changes_nothing(long_model, dtype):
    """Captured decode steps are keyed by (batch size, length class): a request that grows from 500 to 530
    tokens leaves the class of 512 for that of 1,024. Every logits row is compared, and both graphs replay."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    page, vocab = long_model["page"], long_model["cfg"]["vocab_size"]
    g = torch.Generator().manual_seed(512)
    tokens = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in (530, 60)]
    want = [plain.forward(long_model["config"], long_model["weights"], t) for t in tokens]
    model = load_model(long_model["folder"], dtype=dtype, device="cuda:0")
    cache = CacheManager(model.cache_layout(), page, 64, 2, dtype=dtype, device=model.device, prefix_cache=False,
                         max_request_tokens=8192)
    stepper = Stepper(model, cache, max_step_tokens=512, max_step_seqs=2)
    seqs = [cache.open("long"), cache.open("short")]
    stepper.step([StepEntry(seqs[0], tokens[0][:500], []), StepEntry(seqs[1], tokens[1][:30], [])])
    for s in range(30):
        got = stepper.step([StepEntry(seqs[0], [tokens[0][500 + s]], [0]), StepEntry(seqs[1], [tokens[1][30 + s]], [0])]).cpu()
        for r, (i, pos) in enumerate(((0, 500 + s), (1, 30 + s))):
            w = want[i][pos]
            if dtype == "float32":
                assert torch.allclose(got[r], w, atol=5e-6, rtol=2e-5), (i, pos)
            else:
                assert float((got[r] - w).abs().max()) <= 0.02 * float(w.abs().max()), (i, pos)
    assert sorted(stepper._graphs) == [(2, 512), (2, 1024)]
    assert stepper.graph_replays == 30 - 2                 # the first step of each class runs eagerly, the next is captured
    stepper.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_are_bounded_and_outlive_a_larger_prompt_portion(long_model, dtype):
    """The table of captured decode steps keeps at most `max_graphs` entries (the least recently replayed one
    goes first and is captured again when its batch size returns), and a prompt portion that grows a scratch
    buffer which only portions use leaves the captured decode steps alone. Every decode row is compared."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    page, vocab = long_model["page"], long_model["cfg"]["vocab_size"]
    g = torch.Generator().manual_seed(96)
    tokens = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in (70, 45, 52, 400)]
    want = [plain.forward(long_model["config"], long_model["weights"], t) for t in tokens]
    model = load_model(long_model["folder"], dtype=dtype, device="cuda:0")
    cache = CacheManager(model.cache_layout(), page, 64, 4, dtype=dtype, device=model.device, prefix_cache=False,
                         max_request_tokens=1024)
    stepper = Stepper(model, cache, max_step_tokens=512, max_step_seqs=4, max_graphs=2)
    seqs = [cache.open(i) for i in range(4)]
    at = [30, 20, 25]
    stepper.step([StepEntry(seqs[i], tokens[i][:at[i]], []) for i in range(3)])

    def decode(live):
        got = stepper.step([StepEntry(seqs[i], [tokens[i][at[i]]], [0]) for i in live]).cpu()
        for r, i in enumerate(live):
            w = want[i][at[i]]
            if dtype == "float32":
                assert torch.allclose(got[r], w, atol=5e-6, rtol=2e-5), (live, i, at[i])
            else:
                assert float((got[r] - w).abs().max()) <= 0.02 * float(w.abs().max()), (live, i, at[i])
            at[i] += 1

    for live in ([0, 1, 2], [0, 1], [2]):                       # three batch sizes, room for two captures
        for _ in range(3):
            decode(live)
    assert list(stepper._graphs) == [(2, 512), (1, 512)]
    kept = stepper._graphs[(1, 512)]
    # a prompt portion larger than any before: scratch buffers of its own may grow, the captured steps stay
    generation = stepper.workspace.generation
    got = stepper.step([StepEntry(seqs[3], tokens[3][:333], [332])]).cpu()
    assert float((got[0] - want[3][332]).abs().max()) <= (1e-4 if dtype == "float32" else 0.02 * float(want[3][332].abs().max()))
    stepper.workspace.get("a buffer no captured step holds", (1 << 16,), torch.float32)
    assert stepper.workspace.generation != generation
    replays = stepper.graph_replays
    decode([2])
    assert stepper._graphs[(1, 512)] is kept and stepper.graph_replays == replays + 1
    # a buffer that the captured step does hold is allocated anew: that capture is stale and is made again
    (tag, buffer_dtype), _ = next(iter(kept.buffers.items()))
    stepper.workspace.get(tag, (stepper.workspace.buffers[tag, buffer_dtype].numel() + 64,), buffer_dtype)
    decode([2])
    assert stepper._graphs[(1, 512)] is not kept and list(stepper._graphs) == [(2, 512), (1, 512)]
    decode([2])
    for _ in range(3):
        decode([0, 1, 2])                                       # evicted before: warm already, so captured at once
    assert list(stepper._graphs) == [(1, 512), (3, 512)]
    decode([0, 1])
    decode([0, 1])
    assert list(stepper._graphs) == [(3, 512), (2, 512)]
    stepper.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_of_33000_tokens_through_the_engine(long_model, dtype, device):
    """Positions up to 33,000 (rotation angles of thousands of turns), block tables two thousand pages wide,
    prompt portions of 2,048 tokens behind a long history (their keys are cut into chunks for separate
    workgroups), then single tokens over 33,000 keys in as many ranges as the launcher picks. The plain
    implementation runs on the device for this (a 33,000 x 33,000 score matrix per head)."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    page, vocab = long_model["page"], long_model["cfg"]["vocab_size"]
    n, n_decode = 33000, 4
    import json
    cfg = dict(long_model["cfg"], max_position_embeddings=40000)
    (long_model["folder"] / "config.json").write_text(json.dumps(cfg))
    g = torch.Generator().manual_seed(33)
    tokens = torch.randint(0, vocab, (n + n_decode,), generator=g).tolist()
    rows = [0, 2047, 2048, 20479, 20480, n - 1] + list(range(n, n + n_decode))
    w = {k: t.to(device) for k, t in long_model["weights"].items()}
    with torch.device(device):
        want = plain.forward(long_model["config"], w, tokens)[rows].cpu()
    del w
    torch.cuda.empty_cache()
    model = load_model(long_model["folder"], dtype=dtype, device="cuda:0")
    cache = CacheManager(model.cache_layout(), page, (n + n_decode) // page + 2, 1, dtype=dtype, device=model.device,
                         prefix_cache=False, max_request_tokens=n + n_decode + page)
    stepper = Stepper(model, cache, max_step_tokens=2048, max_step_seqs=1)
    seq = cache.open("far")
    got = {}
    for a in range(0, n, 2048):
        b = min(n, a + 2048)
        wanted = [r - a for r in rows if a <= r < b]
        out = stepper.step([StepEntry(seq, tokens[a:b], wanted)]).cpu()
        for j, r in enumerate(wanted):
            got[r + a] = out[j].clone()
    for p in range(n, n + n_decode):
        got[p] = stepper.step([StepEntry(seq, [tokens[p]], [0])]).cpu()[0].clone()
    worst = 0.0
    for j, r in enumerate(rows):
        err = float((got[r] - want[j]).abs().max())
        worst = max(worst, err)
        if dtype == "float32":
            assert torch.allclose(got[r], want[j], atol=5e-6, rtol=2e-5), (r, err)
        else:
            assert err <= 0.02 * float(want[j].abs().max()), (r, err)
    print(f"33,000 tokens, {dtype}: worst difference {worst:.3e}")
    cache.close(seq)
    stepper.close()
