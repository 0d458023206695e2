"""The engine on the GPU: generation through the entry point, long decoding, sampling, prefix reuse,
each part alone, schedules that name a layer twice or share a cache, and a toy mixer with its own state."""
import dataclasses
import json
import math

import pytest
import torch

import plain_model as plain
from tiny_configs import TINY, make_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=["A", "B", "C"])
def tiny(request, tmp_path_factory, device):
    name = request.param
    folder = tmp_path_factory.mktemp(f"eng{name}")
    cfg, page = make_folder(folder, name)
    config, weights = plain.read_folder(folder)
    return dict(name=name, folder=folder, page=page, cfg=cfg, config=config, weights=weights)


def prompts_for(tiny, lengths, seed=5):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, tiny["cfg"]["vocab_size"], (n,), generator=g).tolist() for n in lengths]


def engine(tiny, dtype="float32", **kw):
    from tessweave_engine_amd.cli import engine_for
    options = dict(dtype=dtype, block_size=tiny["page"], kv_blocks=128, max_context=256, prefill_chunk=13,
                   max_active=4, no_prefix_cache=True)
    options.update(kw)
    return engine_for(tiny["folder"], **options)


def test_greedy_generation_through_the_entry_point(tiny):
    """The workloads of the two tiny configurations: ragged prompts, portions of 13 beside decode tokens."""
    lengths, count = ([5, 17, 33], 16) if tiny["name"] == "A" else ([1, 9, 40, 64, 100], 24)
    prompts = prompts_for(tiny, lengths)
    want = [plain.greedy(tiny["config"], tiny["weights"], p, count) for p in prompts]
    e = engine(tiny)
    got = e.generate(prompts, max_tokens=count, ignore_eos=True)
    stats = e.stats()
    e.close()
    assert got == want
    assert stats["graph_replays"] > 0 and stats["free_blocks"] == stats["physical_blocks"]
    # the same through the unpacked projections (the --unfused ablation) and without graphs
    e = engine(tiny, unfused=True, no_graphs=True)
    assert e.generate(prompts[:2], max_tokens=6, ignore_eos=True) == [w[:6] for w in want[:2]]
    e.close()


def test_bfloat16_generation_agrees_where_the_choice_is_clear(tiny):
    prompts = prompts_for(tiny, [7, 30], seed=9)
    e = engine(tiny, dtype="bfloat16")
    got = e.generate(prompts, max_tokens=8, ignore_eos=True)
    e.close()
    clear = total = 0
    for p, out in zip(prompts, got):
        tokens = list(p)
        for t in out:
            logits = plain.forward(tiny["config"], tiny["weights"], tokens)[-1]
            top = logits.topk(2).values
            total += 1
            if float(top[0] - top[1]) > 0.04 * float(logits.abs().max()):
                clear += 1
                assert t == int(logits.argmax())
            tokens.append(t)
    print(f"tiny {tiny['name']}: {clear} of {total} generated tokens had a clear choice and were compared")
    assert clear >= total // 4, (clear, total)       # otherwise this test would compare nothing


def test_long_decoding_and_the_first_tokens(tiny):
    """One token after the other for hundreds of steps (pages fill and new ones are taken), from position 0."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    n = 300
    tokens = prompts_for(tiny, [n], seed=21)[0]
    want = plain.forward(tiny["config"], tiny["weights"], tokens)
    for dtype in ("float32", "bfloat16"):
        model = load_model(tiny["folder"], dtype=dtype, device="cuda:0")
        cache = CacheManager(model.cache_layout(), tiny["page"], math.ceil(n / tiny["page"]), 2, dtype=dtype,
                             device=model.device, prefix_cache=False, max_request_tokens=n + tiny["page"])
        stepper = Stepper(model, cache, max_step_tokens=16)
        seq = cache.open("long")
        rows = [stepper.step([StepEntry(seq, [t], [0])]).cpu().clone() for t in tokens]
        got = torch.cat(rows)
        assert stepper.graph_replays >= n - 2
        if dtype == "float32":
            torch.testing.assert_close(got, want, atol=5e-6, rtol=2e-5)
            torch.testing.assert_close(got[:3], want[:3], atol=5e-6, rtol=2e-5)      # positions 0, 1, 2
        else:
            assert float((got - want).abs().max()) <= 0.02 * float(want.abs().max())
        cache.close(seq)
        cache.check()
        stepper.close()


def test_a_cache_full_of_nan_changes_nothing(tiny):
    """Every page starts as NaN, as memory that is only reserved may: pages a request does not own and the
    unused tail of its last page are never read into a result (the kernels' loads carry no predicate, so
    this is the masks' work). Prompt portions, single tokens and a mixed batch, both precisions."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.weights import load_model
    page = tiny["page"]
    a_tokens, b_tokens = prompts_for(tiny, [2 * page + 3, page + 1], seed=33)
    want = {"a": plain.forward(tiny["config"], tiny["weights"], a_tokens),
            "b": plain.forward(tiny["config"], tiny["weights"], b_tokens)}
    for dtype in ("float32", "bfloat16"):
        model = load_model(tiny["folder"], dtype=dtype, device="cuda:0")
        cache = CacheManager(model.cache_layout(), page, 12, 2, dtype=dtype, device=model.device, prefix_cache=False,
                             max_request_tokens=4 * page)
        for pool in cache.storage:
            pool.fill_(float("nan"))
        stepper = Stepper(model, cache, max_step_tokens=64, use_graphs=False)
        a, b = cache.open("a"), cache.open("b")
        got = {"a": [], "b": []}

        def run(*items):
            entries = [StepEntry(seq, toks[lo:hi], list(range(hi - lo))) for _, seq, toks, lo, hi in items]
            out, row = stepper.step(entries).cpu(), 0
            for name, _, _, lo, hi in items:
                got[name].append(out[row:row + hi - lo].clone())
                row += hi - lo
        run(("a", a, a_tokens, 0, page - 1))                              # ends inside the first page
        run(("a", a, a_tokens, page - 1, page + 2), ("b", b, b_tokens, 0, 1))   # crosses a page edge beside a first token
        run(("b", b, b_tokens, 1, page + 1), ("a", a, a_tokens, page + 2, page + 3))
        for t in range(page + 3, len(a_tokens)):
            run(("a", a, a_tokens, t, t + 1))
        for name in got:
            have = torch.cat(got[name])
            assert torch.isfinite(have).all(), (tiny["name"], dtype, name)
            if dtype == "float32":
                torch.testing.assert_close(have, want[name], atol=5e-6, rtol=2e-5)
            else:
                assert float((have - want[name]).abs().max()) <= 0.02 * float(want[name].abs().max())
        stepper.close()


def test_sampling_seed_is_independent_of_other_requests(tiny):
    """tests/test_engine.py:251-260 of the reference, with the device sampler."""
    p = prompts_for(tiny, [5, 4], seed=2)
    e = engine(tiny)
    a = e.submit(p[0], 7, temperature=.8, seed=9, ignore_eos=True)
    e.drain()
    e.submit(p[1], 9, temperature=.5, seed=8, ignore_eos=True)
    b = e.submit(p[0], 7, temperature=.8, seed=9, ignore_eos=True)
    c = e.submit(p[0], 7, temperature=.8, seed=10, ignore_eos=True)
    e.drain()
    assert a.output == b.output and len(a.output) == 7
    assert c.output != a.output                      # another seed, another stream (7 draws at T=0.8)
    cold = e.submit(p[0], 7, temperature=1e-4, seed=3, ignore_eos=True)
    e.drain()
    assert cold.output == plain.greedy(tiny["config"], tiny["weights"], p[0], 7)
    e.close()


def test_lookahead_and_reading_every_turn_give_the_same_tokens(tiny):
    """Turns put on the device before the last turn's tokens are read (the default) against reading every turn:
    greedy and sampled requests, staggered arrivals, and a request that ends on EOS one turn before the host knows."""
    prompts = prompts_for(tiny, [3, 21, 40, 8], seed=31)
    greedy = plain.greedy(tiny["config"], tiny["weights"], prompts[0], 12)
    first = {}
    for i, t in enumerate(greedy):
        first.setdefault(t, i)
    eos = max(first, key=first.get)                  # the token that first appears latest ends the request there
    outs = []
    for look in (True, False):
        e = engine(tiny, no_lookahead=not look)
        assert e.lookahead == look
        e.model_config = dataclasses.replace(e.model_config, eos_token_ids=(eos,))
        rs = [e.submit(prompts[0], 12), e.submit(prompts[1], 9, temperature=0.7, seed=4, ignore_eos=True)]
        for _ in range(3):
            e.step()
        rs += [e.submit(prompts[2], 5, ignore_eos=True), e.submit(prompts[3], 11, temperature=1.3, seed=6, ignore_eos=True)]
        e.drain()
        outs.append([(r.output, r.status) for r in rs])
        stats = e.stats()
        assert stats["free_blocks"] == stats["physical_blocks"]
        e.close()
    assert outs[0] == outs[1]
    assert outs[0][0] == (greedy[:greedy.index(eos) + 1], "stop")
    assert outs[0][2] == (plain.greedy(tiny["config"], tiny["weights"], prompts[2], 5), "length")


def test_many_requests_with_few_pages_give_the_same_tokens_with_and_without_lookahead(tiny):
    """A few hundred turns of serving in 32-bit, where rounding cannot flip a choice: random prompt lengths,
    temperatures, arrivals, cancellations and two EOS ids, with so few pages that requests wait for them and
    prefix pages are evicted. The tokens of every request are the same in both modes, and no page is lost."""
    import random
    rng = random.Random(7)
    vocab = tiny["cfg"]["vocab_size"]
    plans = [dict(prompt=[rng.randrange(vocab) for _ in range(rng.choice([1, 3, 9, 31, 64, 100]))],
                  max_tokens=rng.choice([1, 2, 7, 20, 40]), temperature=rng.choice([0.0, 0.0, 0.8, 1.5]),
                  gap=rng.choice([0, 0, 1, 3]), cancel_after=rng.randrange(2, 30) if rng.random() < 0.1 else None)
             for _ in range(150)]
    pages = 2 * -(-(100 + 40 + 48) // tiny["page"]) + 3
    outs = []
    for look in (True, False):
        e = engine(tiny, no_lookahead=not look, kv_blocks=pages, max_context=256, prefill_chunk=48, max_active=6,
                   no_prefix_cache=False)
        e.model_config = dataclasses.replace(e.model_config, eos_token_ids=(17, vocab - 2))
        live, cancel, nxt, wait, turn = {}, {}, 0, 0, 0
        while nxt < len(plans) or e.requests:
            while nxt < len(plans) and wait <= 0 and len(e.waiting) < 8:
                p = plans[nxt]
                live[nxt] = e.submit(p["prompt"], p["max_tokens"], temperature=p["temperature"], seed=nxt)
                if p["cancel_after"]:
                    cancel[turn + p["cancel_after"]] = live[nxt].id
                wait, nxt = p["gap"], nxt + 1
            if turn in cancel:
                e.cancel(cancel[turn])
            e.step()
            wait, turn = wait - 1, turn + 1
            if turn % 64 == 0:
                e.cache.check()
            assert turn < 20000
        e.flush()
        e.cache.check()
        outs.append({i: (r.status, tuple(r.output)) for i, r in live.items()})
        e.close()
    differ = [i for i in outs[0] if outs[0][i] != outs[1][i] and "cancelled" not in (outs[0][i][0], outs[1][i][0])]
    assert not differ, [(outs[0][i], outs[1][i]) for i in differ[:3]]
    assert sum(v[0] == "stop" for v in outs[0].values()) >= 1


def test_bfloat16_with_and_without_lookahead_agrees_until_the_first_close_call(tiny):
    """In bfloat16 the two ways of reading tokens may compose batches differently (lookahead retires a request one
    turn later), so a token may be computed beside a prompt portion in one and alone in the other, by kernels
    that sum in another order. That can only matter where the choice is close: a request's tokens must be equal
    up to the first output token at which the plain logits' best two lie within 2 % of the largest logit of
    each other (greedy; bfloat16 logits are themselves held to 2 % of the largest), or at which the draw falls
    within 0.01 of an edge of its word's interval (sampled); from there on the two runs are different sequences
    and are not compared. With random weights the logits are nearly flat, so a request's first close call comes
    early: an eighth of all tokens must still be compared."""
    import random
    from tessweave_engine_amd.kernels import ops
    rng = random.Random(11)
    vocab = tiny["cfg"]["vocab_size"]
    plans = [dict(prompt=[rng.randrange(vocab) for _ in range(rng.choice([1, 3, 9, 31, 64, 100]))],
                  max_tokens=rng.choice([2, 7, 20]), temperature=rng.choice([0.0, 0.0, 0.8]), gap=rng.choice([0, 1, 3]))
             for _ in range(40)]
    outs = []
    for look in (True, False):
        e = engine(tiny, dtype="bfloat16", no_lookahead=not look, kv_blocks=64, max_context=256, prefill_chunk=48,
                   max_active=6)
        live, nxt, wait, turn = {}, 0, 0, 0
        while nxt < len(plans) or e.requests:
            while nxt < len(plans) and wait <= 0 and len(e.waiting) < 8:
                p = plans[nxt]
                live[nxt] = e.submit(p["prompt"], p["max_tokens"], temperature=p["temperature"], seed=nxt, ignore_eos=True)
                wait, nxt = p["gap"], nxt + 1
            e.step()
            wait, turn = wait - 1, turn + 1
            assert turn < 5000
        e.flush()
        outs.append({i: list(r.output) for i, r in live.items()})
        e.close()
    compared = total = 0
    for i, p in enumerate(plans):
        a, b = outs[0][i], outs[1][i]
        assert len(a) == len(b) == p["max_tokens"]
        total += len(a)
        tokens = list(p["prompt"])
        for n, (x, y) in enumerate(zip(a, b)):
            logits = plain.forward(tiny["config"], tiny["weights"], tokens)[-1]
            if p["temperature"] == 0.0:
                top = logits.topk(2).values
                close = float(top[0] - top[1]) <= 0.02 * float(logits.abs().max())
            else:
                cdf = torch.cumsum(plain.softmax_temperature(logits, p["temperature"]).double(), 0)
                target = ops.sampling_uniform(i, n) * float(cdf[-1])
                w = int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))
                close = min(target - (float(cdf[w - 1]) if w else 0.0), float(cdf[w]) - target) < 0.01
            if close:
                break
            assert x == y, (i, n, x, y)
            compared += 1
            tokens.append(x)
    print(f"tiny {tiny['name']}: {compared} of {total} tokens compared between the two ways of reading")
    assert compared >= total // 8, (compared, total)


def test_prefix_pages_are_reused_on_the_gpu(tiny):
    page = tiny["page"]
    shared = prompts_for(tiny, [32], seed=4)[0]
    p1, p2 = shared + [3, 4, 5], shared + [9, 1]
    e = engine(tiny, no_prefix_cache=False)
    first = e.submit(p1, 6, ignore_eos=True)
    e.drain()
    again = e.submit(p1, 6, ignore_eos=True)
    other = e.submit(p2, 6, ignore_eos=True)
    e.drain()
    assert again.cached == 32 and other.cached == 32          # 32 tokens = full pages at both page sizes
    assert again.output == first.output == plain.greedy(tiny["config"], tiny["weights"], p1, 6)
    assert other.output == plain.greedy(tiny["config"], tiny["weights"], p2, 6)
    e.close()
    e.cache.check()
    assert len(e.cache.pools[0].free) == e.cache.pools[0].capacity


def test_requests_that_run_together_share_the_blocks_of_a_common_prompt(tiny):
    """The full blocks of a prompt enter the prefix index as soon as their step has been issued: a request
    that arrives while the first one is still in its prompt or decoding takes them (its own step runs later
    on the same stream), in both ways of reading tokens, and generates what the plain implementation does."""
    shared = prompts_for(tiny, [64], seed=8)[0]
    p1, p2, p3 = shared + [3, 4, 5], shared + [9, 1], shared[:32] + [7, 7, 7]
    want = [plain.greedy(tiny["config"], tiny["weights"], p, 8) for p in (p1, p2, p3)]
    for look in (True, False):
        e = engine(tiny, no_prefix_cache=False, no_lookahead=not look, prefill_chunk=32)
        a = e.submit(p1, 8, ignore_eos=True)
        e.step()                                         # a's first 32 prompt tokens are on the device
        b = e.submit(p2, 8, ignore_eos=True)
        e.step()                                         # b is admitted: it shares what a has issued so far
        e.step()
        c = e.submit(p3, 8, ignore_eos=True)
        e.drain()
        e.flush()
        assert a.cached == 0 and b.cached == 32 and c.cached == 32, (a.cached, b.cached, c.cached)
        assert [a.output, b.output, c.output] == want
        assert e.stats()["prefix_hit_tokens"] == 64
        e.close()
        e.cache.check()
        assert len(e.cache.pools[0].free) == e.cache.pools[0].capacity


# ---- each part alone --------------------------------------------------------------------------------
class PartHarness:
    """A cache, a step context and the GPU stream for running single parts on given sequences."""

    def __init__(self, model, page, dtype):
        from tessweave_engine_amd.cache import CacheManager
        from tessweave_engine_amd.engine import Stepper
        self.cache = CacheManager(model.cache_layout(), page, 64, 4, dtype=dtype, device=model.device,
                                  prefix_cache=False, max_request_tokens=256)
        self.stepper = Stepper(model, self.cache, max_step_tokens=64, use_graphs=False)

    def context(self, entries):
        ctx, ordered, _ = self.stepper.prepare(entries)
        self.stepper.upload(ctx)
        return ctx, ordered


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_part_alone(tiny, dtype):
    from tessweave_engine_amd.engine import StepEntry
    from tessweave_engine_amd.parts import LayerRun, fold_pending
    from tessweave_engine_amd.weights import load_model
    model = load_model(tiny["folder"], dtype=dtype, device="cuda:0")
    torch_dtype = model.dtype
    s, w = plain.sizes(tiny["config"]), tiny["weights"]
    h = PartHarness(model, tiny["page"], dtype)
    a, b = h.cache.open("a"), h.cache.open("b")
    toks = prompts_for(tiny, [11, 6], seed=8)
    tight = dict(atol=2e-5, rtol=2e-5) if dtype == "float32" else dict(atol=3e-2, rtol=3e-2)
    with torch.cuda.stream(h.stepper.stream):
        ctx, ordered = h.context([StepEntry(a, toks[0], []), StepEntry(b, toks[1], [])])
        n = ctx.n_tokens
        # embedding
        x = model.embedding.forward(ctx)
        ids = torch.tensor(toks[0] + toks[1])
        torch.testing.assert_close(x.cpu(), w["model.embed_tokens.weight"][ids], atol=0, rtol=0)
        # norm
        block = model.blocks[0]
        x0 = torch.randn(n, s["hidden"], generator=torch.Generator().manual_seed(1))
        xd = x0.to("cuda")
        hn = block.mixer_norm.forward(ctx, xd)
        want_h = plain.rms_norm(x0, w["model.layers.0.input_layernorm.weight"], s["eps"])
        torch.testing.assert_close(hn.float().cpu(), want_h, **tight)
        # position encoding
        cos, sin = block.mixer.position.tables(ctx)
        pos = torch.cat([torch.arange(11), torch.arange(6)]).float()
        inv = s["theta"] ** (-torch.arange(0, s["head_dim"], 2, dtype=torch.float32) / s["head_dim"])
        torch.testing.assert_close(cos.cpu(), (pos[:, None] * inv).cos(), atol=2e-6, rtol=0)
        torch.testing.assert_close(sin.cpu(), (pos[:, None] * inv).sin(), atol=2e-6, rtol=0)
        # mixer: adds attention of the normalised input into the residual stream
        h_in = want_h.to(torch_dtype)
        xr = xd.clone()
        fold_pending(xr, block.mixer.forward(ctx, LayerRun(0, 0), h_in.to("cuda"), xr))
        want_x = x0.clone()
        want_x[:11] += plain.attention_block(h_in.float()[:11], torch.arange(11), w, "model.layers.0.self_attn.", s)
        want_x[11:] += plain.attention_block(h_in.float()[11:], torch.arange(6), w, "model.layers.0.self_attn.", s)
        torch.testing.assert_close(xr.cpu(), want_x, **tight)
        # feed-forward
        xf = xd.clone()
        fold_pending(xf, block.ffn.forward(ctx, h_in.to("cuda"), xf))
        p = "model.layers.0.mlp."
        want_f = x0 + plain.swiglu(h_in.float(), w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
        torch.testing.assert_close(xf.cpu(), want_f, **tight)
        # whole block
        xb = xd.clone()
        fold_pending(xb, block.forward(ctx, LayerRun(0, 0), xb))
        want_b = torch.cat([plain.decoder_layer(x0[:11], torch.arange(11), w, 0, s),
                            plain.decoder_layer(x0[11:], torch.arange(6), w, 0, s)])
        torch.testing.assert_close(xb.cpu(), want_b, **(tight if dtype == "float32" else dict(atol=6e-2, rtol=6e-2)))
        # head on chosen rows
        rows = torch.tensor([0, n - 1], dtype=torch.int32, device="cuda")
        hf = model.final_norm.forward(ctx, xd, rows=rows)
        logits = model.head.forward(ctx, hf)
        head_w = w["model.embed_tokens.weight"] if s["tied"] else w["lm_head.weight"]
        want_l = plain.rms_norm(x0[[0, n - 1]], w["model.norm.weight"], s["eps"]) @ head_w.T
        torch.testing.assert_close(logits.cpu(), want_l, **(dict(atol=1e-4, rtol=1e-4) if dtype == "float32" else dict(atol=.15, rtol=.05)))
    torch.cuda.synchronize()


# ---- schedules: a layer named twice, a layer that reads another layer's cache --------------------------
def test_schedule_names_a_layer_twice_and_shares_a_cache(tiny):
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.config import build_model, config_from_dict
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.parts import LayerRun
    from tessweave_engine_amd.weights import read_tensors
    cfg = config_from_dict(tiny["cfg"])
    model = build_model(cfg)
    last = len(model.blocks) - 1
    # block 0 runs twice (each run with a cache slot of its own); the last run reuses block `last`
    # but READS the keys and values that the second run of block 0 wrote
    model.schedule = [LayerRun(0, 0), LayerRun(0, 1), LayerRun(last, 1, writes_cache=False)]
    model._layout = None
    model.bind(read_tensors(tiny["folder"], model.tensor_specs(), torch.float32, "cuda:0"), torch.float32, "cuda:0")
    assert len(model.cache_layout().needs) == 2
    s, w = plain.sizes(tiny["config"]), tiny["weights"]
    tokens = prompts_for(tiny, [23], seed=6)[0]

    def plain_run(tokens):
        x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        pos = torch.arange(len(tokens))
        x = plain.decoder_layer(x, pos, w, 0, s)
        # second run of block 0: keep its rotated keys and its values for the sharing layer
        p0 = "model.layers.0."
        hn = plain.rms_norm(x, w[p0 + "input_layernorm.weight"], s["eps"])
        t = len(tokens)
        k = (hn @ w[p0 + "self_attn.k_proj.weight"].T + w[p0 + "self_attn.k_proj.bias"]).reshape(t, s["kv_heads"], s["head_dim"])
        v = (hn @ w[p0 + "self_attn.v_proj.weight"].T + w[p0 + "self_attn.v_proj.bias"]).reshape(t, s["kv_heads"], s["head_dim"])
        k = plain.rope(k, pos, s["theta"])
        x = plain.decoder_layer(x, pos, w, 0, s)
        # sharing layer: its own q, the other layer's k and v
        pl = f"model.layers.{last}."
        hn = plain.rms_norm(x, w[pl + "input_layernorm.weight"], s["eps"])
        q = (hn @ w[pl + "self_attn.q_proj.weight"].T + w[pl + "self_attn.q_proj.bias"]).reshape(t, s["heads"], s["head_dim"])
        q = plain.rope(q, pos, s["theta"])
        att = plain.attention(q, k, v, pos).reshape(t, -1) @ w[pl + "self_attn.o_proj.weight"].T
        x = x + att
        hn = plain.rms_norm(x, w[pl + "post_attention_layernorm.weight"], s["eps"])
        x = x + plain.swiglu(hn, w[pl + "mlp.gate_proj.weight"], w[pl + "mlp.up_proj.weight"], w[pl + "mlp.down_proj.weight"])
        x = plain.rms_norm(x, w["model.norm.weight"], s["eps"])
        head = w["model.embed_tokens.weight"] if s["tied"] else w["lm_head.weight"]
        return x @ head.T

    want = plain_run(tokens)
    cache = CacheManager(model.cache_layout(), tiny["page"], 16, 2, dtype="float32", device=model.device,
                         prefix_cache=False, max_request_tokens=64)
    stepper = Stepper(model, cache, max_step_tokens=32)
    seq = cache.open("s")
    outs = [stepper.step([StepEntry(seq, tokens[:9], list(range(9)))]).cpu().clone(),
            stepper.step([StepEntry(seq, tokens[9:20], list(range(11)))]).cpu().clone()]
    outs += [stepper.step([StepEntry(seq, [t], [0])]).cpu().clone() for t in tokens[20:]]
    torch.testing.assert_close(torch.cat(outs), want, atol=5e-6, rtol=2e-5)
    stepper.close()


# ---- a toy mixer with state of its own, defined here, registered and stepped without touching the package ----
def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path, device):
    from dataclasses import dataclass
    from safetensors.torch import save_file
    from tessweave_engine_amd.cache import CacheManager, CacheNeed, FixedState
    from tessweave_engine_amd.config import register_architecture, unregister_architecture
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.parts import (DecoderModel, Mixer, OutputHead, PreNormBlock, RMSNorm, SwiGLU,
                                            TokenEmbedding, LayerRun, GroupedQueryAttention, RotaryEmbedding)
    from tessweave_engine_amd.weights import MATRIX, TensorSpec, load_model, random_tensors

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        vocab_size: int
        hidden_size: int
        intermediate_size: int
        decay: float
        max_position_embeddings: int = 256
        eos_token_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls("ToyDecayForCausalLM", d["vocab_size"], d["hidden_size"], d["intermediate_size"], d["decay"])

        def to_dict(self):
            return dict(architectures=[self.architecture], model_type="toy_decay", vocab_size=self.vocab_size,
                        hidden_size=self.hidden_size, intermediate_size=self.intermediate_size, decay=self.decay)

    class DecayMixer(Mixer):
        """state_t = decay * state_{t-1} + h_t;  output_t = state_t @ W.T.  The state is the request's own."""
        graph_safe = False                      # written with torch operations

        def __init__(self, name, hidden, decay):
            self.name, self.hidden, self.decay = name, hidden, decay

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.hidden, self.hidden), MATRIX)]

        def bind(self, tensors, dtype, device):
            self.weight = tensors.pop(self.name + ".weight").float()

        def cache_need(self):
            return CacheNeed(state=FixedState((self.hidden,), "float32"))

        def forward(self, ctx, run, h, x):
            state = ctx.cache.state[run.cache_slot]
            for s in range(ctx.n_seqs):
                slot = ctx.h_state_slots[s]
                for row in range(ctx.h_q_start[s], ctx.h_q_start[s + 1]):
                    state[slot] = self.decay * state[slot] + h[row].float()
                    x[row] += state[slot] @ self.weight.T

    def build_toy(c):
        emb = TokenEmbedding("emb", c.vocab_size, c.hidden_size)
        rotary = RotaryEmbedding(16, 10000.0)
        blocks = [PreNormBlock(RMSNorm("l0.n1", c.hidden_size, 1e-5), DecayMixer("l0.mix", c.hidden_size, c.decay),
                               RMSNorm("l0.n2", c.hidden_size, 1e-5), SwiGLU("l0.ff.", c.hidden_size, c.intermediate_size)),
                  PreNormBlock(RMSNorm("l1.n1", c.hidden_size, 1e-5),
                               GroupedQueryAttention("l1.att.", c.hidden_size, 2, 1, 16, rotary, qkv_bias=False),
                               RMSNorm("l1.n2", c.hidden_size, 1e-5), SwiGLU("l1.ff.", c.hidden_size, c.intermediate_size))]
        return DecoderModel(c, emb, blocks, RMSNorm("final", c.hidden_size, 1e-5),
                            OutputHead("head", c.vocab_size, c.hidden_size, tied_to=emb),
                            schedule=[LayerRun(0, 0), LayerRun(1, 1), LayerRun(0, 2)])    # the toy layer runs twice

    register_architecture("ToyDecayForCausalLM", "toy_decay", ToyConfig, build_toy)
    try:
        cfg = ToyConfig("ToyDecayForCausalLM", 61, 32, 48, 0.75)
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        tensors = random_tensors(build_toy(cfg).tensor_specs(), 3, std=0.2)
        save_file(tensors, str(tmp_path / "model.safetensors"))
        model = load_model(tmp_path, dtype="float32", device="cuda:0")          # config.json picks the toy class
        assert type(model.blocks[0].mixer).__name__ == "DecayMixer" and not model.graph_safe_model
        layout = model.cache_layout()
        assert layout.state_slots == (0, 2) and len(layout.groups) == 1 and not layout.shares_prefixes

        w = {k: v.float() for k, v in tensors.items()}

        def plain_toy(tokens):
            x = w["emb.weight"][torch.tensor(tokens)]
            pos = torch.arange(len(tokens))

            def toy_layer(x):
                hn = plain.rms_norm(x, w["l0.n1.weight"], 1e-5)
                state, rows = torch.zeros(32), []
                for t in range(len(tokens)):
                    state = 0.75 * state + hn[t]
                    rows.append(state @ w["l0.mix.weight"].T)
                x = x + torch.stack(rows)
                hn = plain.rms_norm(x, w["l0.n2.weight"], 1e-5)
                return x + plain.swiglu(hn, w["l0.ff.gate_proj.weight"], w["l0.ff.up_proj.weight"], w["l0.ff.down_proj.weight"])
            x = toy_layer(x)
            hn = plain.rms_norm(x, w["l1.n1.weight"], 1e-5)
            t = len(tokens)
            q = plain.rope((hn @ w["l1.att.q_proj.weight"].T).reshape(t, 2, 16), pos, 10000.0)
            k = plain.rope((hn @ w["l1.att.k_proj.weight"].T).reshape(t, 1, 16), pos, 10000.0)
            v = (hn @ w["l1.att.v_proj.weight"].T).reshape(t, 1, 16)
            x = x + plain.attention(q, k, v, pos).reshape(t, 32) @ w["l1.att.o_proj.weight"].T
            hn = plain.rms_norm(x, w["l1.n2.weight"], 1e-5)
            x = x + plain.swiglu(hn, w["l1.ff.gate_proj.weight"], w["l1.ff.up_proj.weight"], w["l1.ff.down_proj.weight"])
            x = toy_layer(x)
            return plain.rms_norm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T

        g = torch.Generator().manual_seed(1)
        seqs = {name: torch.randint(0, 61, (n,), generator=g).tolist() for name, n in (("a", 19), ("b", 12), ("c", 9))}
        cache = CacheManager(layout, 8, 8, 2, dtype="float32", device=model.device, max_request_tokens=32)
        stepper = Stepper(model, cache, max_step_tokens=32)
        a, b = cache.open("a"), cache.open("b")
        got = {"a": [], "b": [], "c": []}

        def run(*items):
            entries = [StepEntry(seq, seqs[name][lo:hi], list(range(hi - lo))) for name, seq, lo, hi in items]
            out, row = stepper.step(entries).cpu(), 0
            for name, _, lo, hi in items:
                got[name].append(out[row:row + hi - lo].clone())
                row += hi - lo
        run(("a", a, 0, 7))
        run(("a", a, 7, 8), ("b", b, 0, 5))                 # a decodes beside b's prompt portion
        run(("b", b, 5, 12), ("a", a, 8, 10))
        cache.close(b)                                       # b's state slot and pages go to c
        c = cache.open("c")
        assert c.state_slot == b.state_slot
        run(("a", a, 10, 19), ("c", c, 0, 9))
        for name in seqs:
            torch.testing.assert_close(torch.cat(got[name]), plain_toy(seqs[name]), atol=2e-5, rtol=2e-5)
        assert stepper.graph_replays == 0
        stepper.close()
    finally:
        unregister_architecture("ToyDecayForCausalLM")


# ---- more toy parts defined here: a feed-forward with routing, another position encoding, a windowed layer ----
def test_toy_routed_feed_forward_scaled_partial_rotary_and_a_window(tmp_path, device):
    """Built from outside the package: a feed-forward that routes each token to one of two SwiGLU experts
    (softmax gate, top 1), a position encoding that rotates only half of each head with positions divided
    by a factor, and a layer whose attention sees a window of 12 keys beside a layer that sees all of them
    (two cache groups; the window's pages return while the request runs). Float32, prompt portions and
    decoded tokens of two requests in one batch, against plain formulas written out below."""
    from dataclasses import dataclass
    from safetensors.torch import save_file
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.config import register_architecture, unregister_architecture
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.kernels import ops
    from tessweave_engine_amd.parts import (DecoderModel, FeedForward, GroupedQueryAttention, LayerRun, OutputHead,
                                            PositionEncoding, PreNormBlock, RMSNorm, SwiGLU, TokenEmbedding,
                                            fold_pending)
    from tessweave_engine_amd.weights import VECTOR, TensorSpec, load_model, random_tensors

    H, HEADS, KV, D, ROT, FACTOR, THETA, WINDOW, INTER, VOCAB = 48, 3, 1, 16, 8, 4.0, 1000.0, 12, 40, 53

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str = "ToyRoutedForCausalLM"
        vocab_size: int = VOCAB
        max_position_embeddings: int = 256
        eos_token_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return dict(architectures=[self.architecture], model_type="toy_routed", vocab_size=self.vocab_size)

    class ScaledPartialRotary(PositionEncoding):
        """cos/sin of (position / factor) * theta^(-2j/rot) for the first `rot` elements of a head."""
        graph_safe = False                                     # written with torch operations

        def __init__(self, rot, theta, factor):
            self.rotary_dim, self.theta, self.factor = rot, theta, factor

        def tables(self, ctx):
            hit = ctx.shared.get(("toy-rotary", id(self)))
            if hit is None:
                inv = self.theta ** (-torch.arange(0, self.rotary_dim, 2, dtype=torch.float32, device=ctx.device) / self.rotary_dim)
                angle = (ctx.positions[0].float() / self.factor)[:, None] * inv[None, :]
                hit = ctx.shared[("toy-rotary", id(self))] = (angle.cos().contiguous(), angle.sin().contiguous())
            return hit

    class RoutedSwiGLU(FeedForward):
        """x += p_e(h) * expert_e(h), e = argmax of softmax(router @ h) (lowest index on ties)."""
        graph_safe = False

        def __init__(self, prefix, hidden, inter, experts):
            self.prefix, self.hidden = prefix, hidden
            self.experts = [SwiGLU(f"{prefix}experts.{e}.", hidden, inter) for e in range(experts)]

        def parts(self):
            return list(self.experts)

        def tensor_specs(self):
            router = TensorSpec(self.prefix + "router.weight", (len(self.experts), self.hidden), VECTOR)   # kept in float32
            return [router] + [s for e in self.experts for s in e.tensor_specs()]

        def bind(self, tensors, dtype, device):
            self.router = tensors.pop(self.prefix + "router.weight").float()
            for e in self.experts:
                e.bind(tensors, dtype, device)

        def forward(self, ctx, h, x):
            probs = torch.softmax(h.float() @ self.router.T, -1)            # router logits in float32
            choice = probs.argmax(-1)
            for e, expert in enumerate(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                out = torch.zeros(rows.numel(), self.hidden, dtype=torch.float32, device=x.device)
                fold_pending(out, expert.forward(ctx, h[rows].contiguous(), out))
                x[rows] += probs[rows, e, None] * out
            return None

    def build_toy(c):
        emb = TokenEmbedding("emb", c.vocab_size, H)
        rotary = ScaledPartialRotary(ROT, THETA, FACTOR)
        blocks = [PreNormBlock(RMSNorm(f"l{i}.n1", H, 1e-5),
                               GroupedQueryAttention(f"l{i}.att.", H, HEADS, KV, D, rotary, qkv_bias=(i == 0), window=window),
                               RMSNorm(f"l{i}.n2", H, 1e-5), RoutedSwiGLU(f"l{i}.ff.", H, INTER, 2))
                  for i, window in enumerate((WINDOW, None))]
        return DecoderModel(c, emb, blocks, RMSNorm("final", H, 1e-5), OutputHead("head", c.vocab_size, H, tied_to=emb))

    register_architecture("ToyRoutedForCausalLM", "toy_routed", ToyConfig, build_toy)
    try:
        cfg = ToyConfig()
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        tensors = random_tensors(build_toy(cfg).tensor_specs(), 5, std=0.3)
        save_file(tensors, str(tmp_path / "model.safetensors"))
        model = load_model(tmp_path, dtype="float32", device="cuda:0")
        layout = model.cache_layout()
        assert len(layout.groups) == 2 and not model.graph_safe_model          # a windowed group beside a full one
        w = {k: v.float() for k, v in tensors.items()}

        def rotate(t, pos):
            inv = THETA ** (-torch.arange(0, ROT, 2, dtype=torch.float32) / ROT)
            angle = (pos.float() / FACTOR)[:, None] * inv[None, :]
            cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
            lo, hi, rest = t[..., :ROT // 2], t[..., ROT // 2:ROT], t[..., ROT:]
            return torch.cat((lo * cos - hi * sin, hi * cos + lo * sin, rest), -1)

        def plain_toy(tokens):
            x = w["emb.weight"][torch.tensor(tokens)]
            t, pos = len(tokens), torch.arange(len(tokens))
            used = set()
            for i, window in enumerate((WINDOW, None)):
                p = f"l{i}."
                hn = plain.rms_norm(x, w[p + "n1.weight"], 1e-5)
                q, k, v = (hn @ w[p + f"att.{n}_proj.weight"].T + (w[p + f"att.{n}_proj.bias"] if i == 0 else 0.0) for n in "qkv")
                q, k = rotate(q.reshape(t, HEADS, D), pos), rotate(k.reshape(t, KV, D), pos)
                att = plain.attention(q, k, v.reshape(t, KV, D), pos, window=window)
                x = x + att.reshape(t, HEADS * D) @ w[p + "att.o_proj.weight"].T
                hn = plain.rms_norm(x, w[p + "n2.weight"], 1e-5)
                probs = torch.softmax(hn @ w[p + "ff.router.weight"].T, -1)
                rows = []
                for r in range(t):
                    e = int(probs[r].argmax())
                    used.add((i, e))
                    rows.append(probs[r, e] * plain.swiglu(hn[r:r + 1], w[p + f"ff.experts.{e}.gate_proj.weight"],
                                                            w[p + f"ff.experts.{e}.up_proj.weight"],
                                                            w[p + f"ff.experts.{e}.down_proj.weight"])[0])
                x = x + torch.stack(rows)
            return plain.rms_norm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T, used

        g = torch.Generator().manual_seed(2)
        seqs = {name: torch.randint(0, VOCAB, (n,), generator=g).tolist() for name, n in (("a", 45), ("b", 30))}
        wants = {name: plain_toy(toks) for name, toks in seqs.items()}
        assert set().union(*(u for _, u in wants.values())) == {(0, 0), (0, 1), (1, 0), (1, 1)}   # every routing branch runs
        page = 4
        cache = CacheManager(layout, page, 24, 2, dtype="float32", device=model.device, prefix_cache=False,
                             max_request_tokens=48)
        stepper = Stepper(model, cache, max_step_tokens=32)
        a, b = cache.open("a"), cache.open("b")
        got = {"a": [], "b": []}

        def run(*items):
            entries = [StepEntry(seq, seqs[name][lo:hi], list(range(hi - lo))) for name, seq, lo, hi in items]
            out, row = stepper.step(entries).cpu(), 0
            for name, _, lo, hi in items:
                got[name].append(out[row:row + hi - lo].clone())
                row += hi - lo
        run(("a", a, 0, 17))
        run(("a", a, 17, 18), ("b", b, 0, 11))               # a decodes beside b's prompt portion
        run(("b", b, 11, 30), ("a", a, 18, 19))
        free_before = [len(p.free) for p in cache.pools]
        for t in range(19, 45):
            run(("a", a, t, t + 1))
        for name in seqs:
            torch.testing.assert_close(torch.cat(got[name]), wants[name][0], atol=3e-5, rtol=3e-5)
        # the windowed group gave pages back while request a went on; the full group only took more
        windowed = [g for g, grp in enumerate(layout.groups) if grp.spec.window][0]
        held = [len(a.tables[g]) - sum(1 for p in a.tables[g] if p < 0) for g in range(2)]
        assert held[windowed] <= WINDOW // page + 2 < held[1 - windowed]
        assert len(cache.pools[1 - windowed].free) < free_before[1 - windowed]
        cache.close(a), cache.close(b)
        cache.check()
        stepper.close()
    finally:
        unregister_architecture("ToyRoutedForCausalLM")


def test_a_norm_that_folds_nothing_and_a_rotation_of_adjacent_pairs(tmp_path, device):
    """Two more toy parts, built outside the package: a norm that knows nothing of pending partial sums (the
    model then never defers any) and a rotary encoding that turns elements (2j, 2j + 1) of the first 8 of 16.
    Float32, a prompt in two portions and decoded tokens, against formulas written out here (the kernel behind
    the pairing is compared in both precisions in test_kernels_gpu)."""
    from dataclasses import dataclass
    from safetensors.torch import save_file
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.config import register_architecture, unregister_architecture
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.parts import (DecoderModel, GroupedQueryAttention, Norm, OutputHead, PreNormBlock,
                                            RotaryEmbedding, SwiGLU, TokenEmbedding)
    from tessweave_engine_amd.weights import VECTOR, ONE_PLUS_NORMAL, TensorSpec, load_model, random_tensors

    H, HEADS, KV, D, ROT, THETA, INTER, VOCAB = 32, 2, 1, 16, 8, 100.0, 48, 41

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str = "ToyCenteredForCausalLM"
        vocab_size: int = VOCAB
        max_position_embeddings: int = 128
        eos_token_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return dict(architectures=[self.architecture], model_type="toy_centered", vocab_size=self.vocab_size)

    class CenteredNorm(Norm):
        """(x - mean) / sqrt(var + eps) * weight, written with torch operations; takes no pending sums."""
        graph_safe = False

        def __init__(self, name, size, eps):
            self.name, self.size, self.eps = name, size, eps

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.size,), VECTOR, ONE_PLUS_NORMAL)]

        def bind(self, tensors, dtype, device):
            self.weight, self.dtype = tensors.pop(self.name + ".weight"), dtype

        def forward(self, ctx, x, rows=None):
            if rows is not None:
                x = x[rows.long()]
            c = x - x.mean(-1, keepdim=True)
            return (c * torch.rsqrt(c.square().mean(-1, keepdim=True) + self.eps) * self.weight).to(self.dtype).contiguous()

    def build_toy(c):
        emb = TokenEmbedding("emb", c.vocab_size, H)
        rotary = RotaryEmbedding(D, THETA, rotary_dim=ROT, pairing="adjacent")
        blocks = [PreNormBlock(CenteredNorm(f"l{i}.n1", H, 1e-5),
                               GroupedQueryAttention(f"l{i}.att.", H, HEADS, KV, D, rotary, qkv_bias=True),
                               CenteredNorm(f"l{i}.n2", H, 1e-5), SwiGLU(f"l{i}.ff.", H, INTER)) for i in range(2)]
        return DecoderModel(c, emb, blocks, CenteredNorm("final", H, 1e-5), OutputHead("head", c.vocab_size, H, tied_to=emb))

    register_architecture("ToyCenteredForCausalLM", "toy_centered", ToyConfig, build_toy)
    try:
        cfg = ToyConfig()
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        tensors = random_tensors(build_toy(cfg).tensor_specs(), 9, std=0.3)
        save_file(tensors, str(tmp_path / "model.safetensors"))
        w = {k: v.float() for k, v in tensors.items()}

        def norm(x, weight):
            c = x - x.mean(-1, keepdim=True)
            return c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-5) * weight

        def rotate(t, pos):
            inv = THETA ** (-torch.arange(0, ROT, 2, dtype=torch.float32) / ROT)
            angle = pos.float()[:, None] * inv[None, :]
            cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
            out = t.clone()
            even, odd = t[..., 0:ROT:2], t[..., 1:ROT:2]
            out[..., 0:ROT:2], out[..., 1:ROT:2] = even * cos - odd * sin, odd * cos + even * sin
            return out

        def plain_toy(tokens):
            x = w["emb.weight"][torch.tensor(tokens)]
            t, pos = len(tokens), torch.arange(len(tokens))
            for i in range(2):
                p = f"l{i}."
                hn = norm(x, w[p + "n1.weight"])
                q, k, v = (hn @ w[p + f"att.{n}_proj.weight"].T + w[p + f"att.{n}_proj.bias"] for n in "qkv")
                att = plain.attention(rotate(q.reshape(t, HEADS, D), pos), rotate(k.reshape(t, KV, D), pos),
                                      v.reshape(t, KV, D), pos)
                x = x + att.reshape(t, HEADS * D) @ w[p + "att.o_proj.weight"].T
                hn = norm(x, w[p + "n2.weight"])
                x = x + plain.swiglu(hn, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
            return norm(x, w["final.weight"]) @ w["emb.weight"].T

        tokens = torch.randint(0, VOCAB, (40,), generator=torch.Generator().manual_seed(4)).tolist()
        want = plain_toy(tokens)
        for dtype in ("float32",):
            model = load_model(tmp_path, dtype=dtype, device="cuda:0")
            assert not model.defers_sums and not model.graph_safe_model
            cache = CacheManager(model.cache_layout(), 8, 8, 1, dtype=dtype, device=model.device, prefix_cache=False,
                                 max_request_tokens=48)
            stepper = Stepper(model, cache, max_step_tokens=32)
            seq = cache.open("r")
            got = [stepper.step([StepEntry(seq, tokens[:19], list(range(19)))]).cpu().clone(),
                   stepper.step([StepEntry(seq, tokens[19:30], list(range(11)))]).cpu().clone()]
            got += [stepper.step([StepEntry(seq, [t], [0])]).cpu().clone() for t in tokens[30:]]
            got = torch.cat(got)
            torch.testing.assert_close(got, want, atol=3e-5, rtol=3e-5)
            cache.close(seq)
            stepper.close()
    finally:
        unregister_architecture("ToyCenteredForCausalLM")


def test_toy_attention_with_soft_capped_scores(tmp_path, device):
    """A toy model, built outside the package, whose attention passes its scaled scores through
    cap * tanh(score / cap): one of two layers, with scores several times the cap. Both precisions
    (bfloat16 takes the attention kernels for every type and page size, since the fast ones have no such step),
    a prompt in portions, decoded tokens, two requests in one batch; against the formula written out here."""
    from dataclasses import dataclass
    from safetensors.torch import save_file
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.config import register_architecture, unregister_architecture
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.parts import (DecoderModel, GroupedQueryAttention, OutputHead, PreNormBlock, RMSNorm,
                                            RotaryEmbedding, SwiGLU, TokenEmbedding)
    from tessweave_engine_amd.weights import load_model, random_tensors

    H, HEADS, KV, D, THETA, INTER, VOCAB, CAP = 32, 4, 2, 16, 100.0, 48, 43, 2.0

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str = "ToyCappedForCausalLM"
        vocab_size: int = VOCAB
        max_position_embeddings: int = 128
        eos_token_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return dict(architectures=[self.architecture], model_type="toy_capped", vocab_size=self.vocab_size)

    def build_toy(c):
        emb = TokenEmbedding("emb", c.vocab_size, H)
        rotary = RotaryEmbedding(D, THETA)
        blocks = [PreNormBlock(RMSNorm(f"l{i}.n1", H, 1e-5),
                               GroupedQueryAttention(f"l{i}.att.", H, HEADS, KV, D, rotary, qkv_bias=True,
                                                     softcap=CAP if i == 0 else None),
                               RMSNorm(f"l{i}.n2", H, 1e-5), SwiGLU(f"l{i}.ff.", H, INTER)) for i in range(2)]
        return DecoderModel(c, emb, blocks, RMSNorm("final", H, 1e-5), OutputHead("head", c.vocab_size, H, tied_to=emb))

    register_architecture("ToyCappedForCausalLM", "toy_capped", ToyConfig, build_toy)
    try:
        cfg = ToyConfig()
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        tensors = random_tensors(build_toy(cfg).tensor_specs(), 12, std=0.3)
        save_file(tensors, str(tmp_path / "model.safetensors"))
        biggest = []

        def plain_toy(tokens, w):
            x = w["emb.weight"][torch.tensor(tokens)]
            t, pos = len(tokens), torch.arange(len(tokens))
            for i in range(2):
                p = f"l{i}."
                hn = plain.rms_norm(x, w[p + "n1.weight"], 1e-5)
                q, k, v = (hn @ w[p + f"att.{n}_proj.weight"].T + w[p + f"att.{n}_proj.bias"] for n in "qkv")
                q, k, v = plain.rope(q.reshape(t, HEADS, D), pos, THETA), plain.rope(k.reshape(t, KV, D), pos, THETA), v.reshape(t, KV, D)
                if i == 0:
                    kk, vv = k.repeat_interleave(HEADS // KV, 1), v.repeat_interleave(HEADS // KV, 1)
                    scores = torch.einsum("qhd,khd->hqk", q, kk) * D ** -0.5
                    biggest.append(float(scores.abs().max()))
                    scores = CAP * torch.tanh(scores / CAP)
                    scores = scores.masked_fill(pos[None, None, :] > pos[None, :, None], float("-inf"))
                    att = torch.einsum("hqk,khd->qhd", torch.softmax(scores, -1), vv)
                else:
                    att = plain.attention(q, k, v, pos)
                x = x + att.reshape(t, HEADS * D) @ w[p + "att.o_proj.weight"].T
                hn = plain.rms_norm(x, w[p + "n2.weight"], 1e-5)
                x = x + plain.swiglu(hn, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
            return plain.rms_norm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T

        g = torch.Generator().manual_seed(6)
        seqs = {name: torch.randint(0, VOCAB, (n,), generator=g).tolist() for name, n in (("a", 37), ("b", 21))}
        for dtype in ("float32", "bfloat16"):
            w = {k: (v.to(torch.bfloat16).float() if dtype == "bfloat16" and v.dtype.is_floating_point else v.float())
                 for k, v in tensors.items()}
            wants = {name: plain_toy(toks, w) for name, toks in seqs.items()}
            assert max(biggest) > 3 * CAP                                 # the cap matters
            model = load_model(tmp_path, dtype=dtype, device="cuda:0")
            cache = CacheManager(model.cache_layout(), 8, 12, 2, dtype=dtype, device=model.device, prefix_cache=False,
                                 max_request_tokens=40)
            stepper = Stepper(model, cache, max_step_tokens=32)
            a, b = cache.open("a"), cache.open("b")
            got = {"a": [], "b": []}

            def run(*items):
                entries = [StepEntry(seq, seqs[name][lo:hi], list(range(hi - lo))) for name, seq, lo, hi in items]
                out, row = stepper.step(entries).float().cpu(), 0
                for name, _, lo, hi in items:
                    got[name].append(out[row:row + hi - lo].clone())
                    row += hi - lo
            run(("a", a, 0, 13))
            run(("a", a, 13, 14), ("b", b, 0, 9))                         # a decodes beside b's prompt portion
            run(("b", b, 9, 21), ("a", a, 14, 20))
            for t in range(20, 37):
                run(("a", a, t, t + 1))
            for name in seqs:
                # (bfloat16: the bar of the replay tests, 2 % of the largest logit, absolute)
                tol = dict(atol=3e-5, rtol=3e-5) if dtype == "float32" else dict(atol=0.02 * float(wants[name].abs().max()), rtol=0)
                torch.testing.assert_close(torch.cat(got[name]), wants[name], **tol)
            cache.close(a), cache.close(b)
            cache.check()
            stepper.close()
    finally:
        unregister_architecture("ToyCappedForCausalLM")


def test_toy_position_ids_on_two_axes_a_hook_between_bias_and_rotation_and_the_weights_a_step_reads(tmp_path, device):
    """Three things another architecture may need, built outside the package: an encoding that reads TWO position
    ids per token (half of the rotary pairs turn with each; step entries bring the ids), a per-head RMS norm of q
    and k between the projection's bias and the rotation (a `HeadHook`, in one of two layers), and a count of the
    bytes a step reads that includes the hook's weights because the part names them. Float32, prompt portions and
    decoded tokens of two requests in one batch, one with its own position ids and one without."""
    from dataclasses import dataclass
    from safetensors.torch import save_file
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.config import register_architecture, unregister_architecture
    from tessweave_engine_amd.engine import StepEntry, Stepper
    from tessweave_engine_amd.parts import (DecoderModel, GroupedQueryAttention, HeadHook, OutputHead,
                                            PositionEncoding, PreNormBlock, RMSNorm, SwiGLU, TokenEmbedding)
    from tessweave_engine_amd.weights import VECTOR, ONE_PLUS_NORMAL, TensorSpec, load_model, random_tensors

    H, HEADS, KV, D, THETA, INTER, VOCAB, EPS = 32, 2, 1, 16, 100.0, 48, 48, 1e-5

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str = "ToyTwoAxisForCausalLM"
        vocab_size: int = VOCAB
        max_position_embeddings: int = 128
        eos_token_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return dict(architectures=[self.architecture], model_type="toy_two_axis", vocab_size=self.vocab_size)

    class TwoAxisRotary(PositionEncoding):
        """Pair j of a head turns by ids[0] * theta^(-2j/D) for j < D/4 and by ids[1] * theta^(-2j/D) above."""
        graph_safe = False
        position_axes = 2
        rotary_dim = D

        def tables(self, ctx):
            hit = ctx.shared.get(("two-axis", id(self)))
            if hit is None:
                assert tuple(ctx.positions.shape) == (2, ctx.n_tokens)
                inv = THETA ** (-torch.arange(0, D, 2, dtype=torch.float32, device=ctx.device) / D)
                axis = (torch.arange(D // 2, device=ctx.device) >= D // 4).long()
                angle = ctx.positions.float()[axis, :].T * inv[None, :]              # [n, D/2]
                hit = ctx.shared[("two-axis", id(self))] = (angle.cos().contiguous(), angle.sin().contiguous())
            return hit

    class HeadRMS(HeadHook):
        """q and k heads each divided by their own root mean square and multiplied by a weight; v as it is."""
        graph_safe = False

        def __init__(self, prefix):
            self.prefix = prefix

        def tensor_specs(self):
            return [TensorSpec(self.prefix + f"{n}_norm.weight", (D,), VECTOR, ONE_PLUS_NORMAL) for n in "qk"]

        def bind(self, tensors, dtype, device):
            self.q_weight = tensors.pop(self.prefix + "q_norm.weight")
            self.k_weight = tensors.pop(self.prefix + "k_norm.weight")

        def weight_tensors(self):
            return [self.q_weight, self.k_weight]

        def forward(self, ctx, qkv):
            for first, heads, weight in ((0, HEADS, self.q_weight), (HEADS * D, KV, self.k_weight)):
                view = qkv[:, first:first + heads * D].view(-1, heads, D)
                x = view.float()
                view.copy_((x * torch.rsqrt(x.square().mean(-1, keepdim=True) + EPS) * weight).to(qkv.dtype))

    def build_toy(c):
        emb = TokenEmbedding("emb", c.vocab_size, H)
        rotary = TwoAxisRotary()
        blocks = [PreNormBlock(RMSNorm(f"l{i}.n1", H, EPS),
                               GroupedQueryAttention(f"l{i}.att.", H, HEADS, KV, D, rotary, qkv_bias=True,
                                                     head_hook=HeadRMS(f"l{i}.att.") if i == 0 else None),
                               RMSNorm(f"l{i}.n2", H, EPS), SwiGLU(f"l{i}.ff.", H, INTER)) for i in range(2)]
        return DecoderModel(c, emb, blocks, RMSNorm("final", H, EPS), OutputHead("head", c.vocab_size, H, tied_to=emb))

    register_architecture("ToyTwoAxisForCausalLM", "toy_two_axis", ToyConfig, build_toy)
    try:
        cfg = ToyConfig()
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        tensors = random_tensors(build_toy(cfg).tensor_specs(), 12, std=0.3)
        assert "l0.att.q_norm.weight" in tensors and "l1.att.q_norm.weight" not in tensors
        save_file(tensors, str(tmp_path / "model.safetensors"))
        model = load_model(tmp_path, dtype="float32", device="cuda:0")
        assert model.position_axes == 2 and not model.graph_safe_model
        # every tensor but the embedding's table (a step gathers rows of it; the tied head reads a copy of its own)
        assert model.weight_bytes() == 4 * sum(t.numel() for t in tensors.values())
        w = {k: v.float() for k, v in tensors.items()}

        def rotate(t, ids):
            inv = THETA ** (-torch.arange(0, D, 2, dtype=torch.float32) / D)
            which = torch.cat([ids[0].float()[:, None].expand(-1, D // 4), ids[1].float()[:, None].expand(-1, D // 4)], 1)
            angle = which * inv[None, :]
            cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
            lo, hi = t[..., :D // 2], t[..., D // 2:]
            return torch.cat((lo * cos - hi * sin, hi * cos + lo * sin), -1)

        def head_rms(t, weight):
            return t / torch.sqrt((t * t).mean(-1, keepdim=True) + EPS) * weight

        def plain_toy(tokens, ids):
            x = w["emb.weight"][torch.tensor(tokens)]
            t, order = len(tokens), torch.arange(len(tokens))
            for i in range(2):
                p = f"l{i}."
                hn = plain.rms_norm(x, w[p + "n1.weight"], EPS)
                q, k, v = (hn @ w[p + f"att.{n}_proj.weight"].T + w[p + f"att.{n}_proj.bias"] for n in "qkv")
                q, k = q.reshape(t, HEADS, D), k.reshape(t, KV, D)
                if i == 0:                                   # after the bias, before the rotation
                    q, k = head_rms(q, w[p + "att.q_norm.weight"]), head_rms(k, w[p + "att.k_norm.weight"])
                att = plain.attention(rotate(q, ids), rotate(k, ids), v.reshape(t, KV, D), order)   # causal by token order
                x = x + att.reshape(t, HEADS * D) @ w[p + "att.o_proj.weight"].T
                hn = plain.rms_norm(x, w[p + "n2.weight"], EPS)
                x = x + plain.swiglu(hn, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
            return plain.rms_norm(x, w["final.weight"], EPS) @ w["emb.weight"].T

        g = torch.Generator().manual_seed(6)
        toks = {"a": torch.randint(0, VOCAB, (30,), generator=g).tolist(), "b": torch.randint(0, VOCAB, (14,), generator=g).tolist()}
        # request a brings its own ids: a grid of 4 columns for its first 16 tokens (axis 0 the row, axis 1 the column),
        # then both axes count on from 4; request b brings none: both axes count its tokens
        ids_a = torch.tensor([[r // 4 for r in range(16)] + list(range(4, 18)), [r % 4 for r in range(16)] + list(range(4, 18))])
        ids_b = torch.arange(14)[None].expand(2, -1)
        want = {"a": plain_toy(toks["a"], ids_a), "b": plain_toy(toks["b"], ids_b)}
        # the ids matter: the same tokens with default ids give other logits
        assert (plain_toy(toks["a"], torch.arange(30)[None].expand(2, -1)) - want["a"]).abs().max() > 1e-2
        cache = CacheManager(model.cache_layout(), 8, 12, 2, dtype="float32", device=model.device, prefix_cache=False,
                             max_request_tokens=48)
        stepper = Stepper(model, cache, max_step_tokens=32)
        a, b = cache.open("a"), cache.open("b")
        got = {"a": [], "b": []}

        def run(*items):
            entries = []
            for name, seq, lo, hi in items:
                own = ids_a[:, lo:hi].tolist() if name == "a" else None
                entries.append(StepEntry(seq, toks[name][lo:hi], list(range(hi - lo)), positions=own))
            out, row = stepper.step(entries).cpu(), 0
            for name, _, lo, hi in items:
                got[name].append(out[row:row + hi - lo].clone())
                row += hi - lo
        run(("a", a, 0, 11))
        run(("a", a, 11, 12), ("b", b, 0, 9))                # a decodes beside b's prompt portion
        run(("b", b, 9, 10), ("a", a, 12, 21))
        for t in range(21, 30):
            run(("a", a, t, t + 1), *([("b", b, t - 11, t - 10)] if t - 11 < 14 else []))
        for name in toks:
            torch.testing.assert_close(torch.cat(got[name]), want[name], atol=3e-5, rtol=3e-5)
        with pytest.raises(ValueError, match="positions must be 2 lists"):
            stepper.step([StepEntry(a, [1], [0], positions=[[30]])])
        stepper.close()
    finally:
        unregister_architecture("ToyTwoAxisForCausalLM")
