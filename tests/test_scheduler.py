"""The scheduler's decisions, with a fake step function and sampler (no GPU)."""
import queue

import pytest
import torch

from tessweave_engine_amd.cache import CacheManager, CapacityError
from tessweave_engine_amd.config import EngineConfig, build_model, config_from_dict
from tessweave_engine_amd.engine import Engine

VOCAB = 128
CFG = dict(model_type="qwen2", vocab_size=VOCAB, hidden_size=64, intermediate_size=64, num_hidden_layers=2,
           num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128)


def next_token(history):
    """A deterministic toy language model: the next token is a function of the whole history."""
    return (sum((i + 1) * t for i, t in enumerate(history)) * 7 + len(history)) % VOCAB


class FakeStepper:
    """Keeps each request's tokens as the real cache would, returns one-hot logits, logs every batch."""

    def __init__(self, cache):
        self.cache, self.history, self.batches, self.fail = cache, {}, [], None

    def step(self, entries):
        if self.fail:
            raise self.fail
        rows = []
        self.batches.append([(e.seq.id, e.seq.computed, len(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            self.cache.ensure(e.seq, e.seq.computed + len(e.tokens))
            h = self.history.setdefault(e.seq.id, [None] * 0)
            assert len(h) <= e.seq.computed                          # prefix-shared tokens were never run here
            h.extend([None] * (e.seq.computed - len(h)))
            h.extend(e.tokens)
            for w in e.want:
                rows.append((e, e.seq.computed + w + 1))
        logits = torch.zeros(len(rows), VOCAB)
        for i, (e, upto) in enumerate(rows):
            logits[i, next_token(self.full[e.seq.id][:upto])] = 1.0
        for e in entries:
            self.cache.advance(e.seq, e.seq.computed + len(e.tokens))
        return logits

    full = {}


class FakeSampler:
    def sample(self, logits, temperatures, seeds, counters):
        self.last = (list(temperatures), list(seeds), list(counters))
        return logits.argmax(-1).tolist()


def make(**kw):
    defaults = dict(block_size=4, kv_blocks=32, max_context=64, prefill_chunk=4, min_prefill_chunk=1, dtype="float32")
    defaults.update(kw)
    config = EngineConfig(**defaults)
    model = build_model(config_from_dict(CFG))
    cache = CacheManager(model.cache_layout(), config.block_size, config.kv_blocks, config.max_active,
                         prefix_cache=config.prefix_cache, max_request_tokens=config.max_context)
    stepper = FakeStepper(cache)
    stepper.full = {}
    engine = Engine(model, config, stepper=stepper, cache=cache, sampler=FakeSampler())
    submit = engine.submit

    def tracked(tokens, *a, **k):
        r = submit(tokens, *a, **k)
        stepper.full[r.id] = r.tokens                                  # the request's growing token list
        return r
    engine.submit = tracked
    return engine, stepper


def expected(prompt, n):
    tokens, out = list(prompt), []
    for _ in range(n):
        out.append(next_token(tokens))
        tokens.append(out[-1])
    return out


def drain(engine):
    for _ in range(500):
        if not engine.step():
            return
    raise AssertionError("engine did not terminate")


def test_submit_validation():
    e, _ = make()
    for prompt, count in (([], 1), ([VOCAB], 1), ([1], 64), ([1], 0), ([1.0], 1), ([-1], 1)):
        with pytest.raises(ValueError):
            e.submit(prompt, count)
    for t in (-0.1, 2.5, float("nan"), float("inf")):
        with pytest.raises(ValueError):
            e.submit([1], 1, temperature=t)
    small, _ = make(kv_blocks=2)
    with pytest.raises(ValueError):
        small.submit([1] * 8, 4)                                       # could never fit: refused, not queued
    e.close()


def test_chunked_prompts_decode_and_outputs():
    e, s = make()
    prompts = [[4, 5, 6, 7, 8], [2, 3, 4, 5, 6, 7, 8, 9, 10]]
    rs = [e.submit(p, 7) for p in prompts]
    drain(e)
    for r, p in zip(rs, prompts):
        assert r.output == expected(p, 7) and r.status == "length"
        assert r.events.qsize() == 8
    # every step: decode tokens first, then prompt portions, within the token budget
    for batch in s.batches:
        counts = [c for _, _, c, _ in batch]
        kinds = [c == 1 and bool(w) for _, _, c, w in batch]
        assert sum(counts) <= e.config.step_token_budget
    e.close()
    e.cache.check()
    assert len(e.cache.pools[0].free) == 32


def test_round_robin_and_first_token_from_the_completing_portion():
    e, s = make(max_step_tokens=4, max_active=2)          # room for one portion of 4 per step
    a = e.submit(list(range(1, 11)), 2)                   # 10 tokens: portions 4, 4, 2
    b = e.submit(list(range(20, 29)), 2)                  # 9 tokens: portions 4, 4, 1
    e.step(); e.step(); e.step(); e.step()
    order = [[(rid, start, n) for rid, start, n, _ in batch] for batch in s.batches]
    assert order[0] == [(a.id, 0, 4)] and order[1] == [(b.id, 0, 4)]          # round-robin over the two prompts
    assert order[2] == [(a.id, 4, 4)] and order[3] == [(b.id, 4, 4)]
    assert not a.output and not b.output
    e.step()          # a's last portion (2 tokens) completes its prompt; the budget's rest completes b's
    assert s.batches[4] == [(a.id, 8, 2, [1]), (b.id, 8, 1, [0])]
    assert a.output == expected(a.prompt, 1) and b.output == expected(b.prompt, 1)
    e.step()          # both decode: one token each, logits wanted for both
    assert s.batches[5] == [(a.id, 10, 1, [0]), (b.id, 9, 1, [0])]
    assert a.status == "length" and b.status == "length" and b.output == expected(b.prompt, 2)
    assert not e.step()
    # decode comes first in a mixed step
    e, s = make(max_step_tokens=5, max_active=2)
    a = e.submit([1, 2], 3)
    e.step()
    b = e.submit(list(range(30, 40)), 1)
    e.step()
    assert s.batches[1] == [(a.id, 2, 1, [0]), (b.id, 0, 4, [])]
    e.close()


def test_budget_lets_several_prompts_advance_but_no_crumbs():
    e, s = make(max_step_tokens=16, prefill_chunk=8, min_prefill_chunk=4, max_active=3)
    a, b, c = e.submit([1] * 20, 1), e.submit([2] * 20, 1), e.submit([3] * 20, 1)
    e.step()
    assert [(rid, n) for rid, _, n, _ in s.batches[0]] == [(a.id, 8), (b.id, 8)]      # 16 tokens; nothing left for c
    e, s = make(max_step_tokens=11, prefill_chunk=8, min_prefill_chunk=4, max_active=3)
    a, b = e.submit([1] * 20, 1), e.submit([2] * 20, 1)
    e.step()
    assert [(rid, n) for rid, _, n, _ in s.batches[0]] == [(a.id, 8)]                 # 3 left: below the minimum portion
    e.close()


def test_eos_is_emitted_then_stops_and_ignore_eos():
    prompt = [3, 4, 5, 6, 7]
    want = expected(prompt, 12)
    end = next(i for i in range(2, 12) if want[i] not in want[:i])
    cfg = dict(CFG, eos_token_id=want[end])
    model = build_model(config_from_dict(cfg))
    config = EngineConfig(block_size=4, kv_blocks=32, max_context=64, prefill_chunk=4, min_prefill_chunk=1, dtype="float32")
    cache = CacheManager(model.cache_layout(), 4, 32, 4, max_request_tokens=64)
    s = FakeStepper(cache)
    s.full = {}
    e = Engine(model, config, stepper=s, cache=cache, sampler=FakeSampler())
    r = e.submit(prompt, 12)
    s.full[r.id] = r.tokens
    r2 = e.submit(prompt, 12, ignore_eos=True)
    s.full[r2.id] = r2.tokens
    drain(e)
    assert r.status == "stop" and r.output == want[:end + 1]            # EOS is part of the output
    assert r2.status == "length" and r2.output == want
    done = [ev for ev in iter(lambda: r.events.get_nowait() if not r.events.empty() else None, None)][-1]
    assert done["finish_reason"] == "stop" and done["usage"] == {"prompt_tokens": 5, "completion_tokens": end + 1,
                                                                 "total_tokens": 6 + end}
    e.close()


def test_admission_reserves_the_worst_case_and_waits_in_order():
    # reference vector (tests/test_engine.py:160-170): 4 pages of 4; two requests of 6 + 6 tokens need 3 each
    e, s = make(kv_blocks=4)
    a = e.submit([1, 2, 3, 4, 5, 6], 6)
    b = e.submit([8, 9, 10, 11, 12, 13], 6)
    e.step()
    assert a.status == "active" and b.status == "waiting"
    drain(e)
    assert len(a.output) == 6 and len(b.output) == 6 and b.output == expected(b.prompt, 6)
    # no skipping ahead: a small request behind a large one waits too
    e, s = make(kv_blocks=4, max_active=3)
    first = e.submit([1] * 6, 6)
    large = e.submit([2] * 10, 6)        # 4 pages: cannot be admitted while `first` runs
    small = e.submit([3], 1)             # 1 page would fit, but it is behind `large`
    e.step()
    assert (first.status, large.status, small.status) == ("active", "waiting", "waiting")
    drain(e)
    assert [r.status for r in (first, large, small)] == ["length"] * 3
    e.cache.check()
    e.close()


def test_pages_never_run_out_mid_generation():
    e, s = make(kv_blocks=6, max_active=4)
    rs = [e.submit([i + 1] * 5, 7) for i in range(4)]          # 3 pages each: two at a time
    while e.step():
        e.cache.check()
        assert len(e.active) <= 2
    assert all(r.status == "length" and len(r.output) == 7 for r in rs)
    e.close()


def test_prefix_reuse_vectors():
    # tests/test_engine.py:113-126 of the reference: cached == 8, one prompt token runs, same output
    e, s = make()
    p = [2, 3, 4, 5, 6, 7, 8, 9, 10]
    first = e.submit(p, 5)
    drain(e)
    count = e.counters["prefill_tokens"]
    second = e.submit(p, 5)
    drain(e)
    assert first.output == second.output and second.cached == 8
    assert e.counters["prefill_tokens"] - count == 1
    # :128-137: a divergent tail shares only the full block before it
    third = e.submit([2, 3, 4, 5, 60, 70], 4)
    drain(e)
    assert third.cached == 4 and third.output == expected(third.prompt, 4)
    # :139-147: another namespace shares nothing
    fourth = e.submit(p, 2, namespace="tenant-b")
    drain(e)
    assert fourth.cached == 0
    e.close()
    e.cache.check()
    assert len(e.cache.pools[0].free) == e.cache.pools[0].capacity


def test_cancel_queue_limit_and_slow_consumer():
    e, s = make(max_active=1)
    a = e.submit([1, 2, 3, 4, 5, 6, 7], 8)
    b = e.submit([1, 2], 8)
    e.step()
    e.cancel(b.id)
    e.cancel(a.id)
    assert not e.step() and (a.status, b.status) == ("cancelled", "cancelled")
    pool = e.cache.pools[0]
    # a's first full prompt block was computed and entered into the prefix index before the cancel: it stays
    # there, evictable; everything else is free
    assert len(pool.prefixes) == 1 and len(pool.free) == pool.capacity - 1 and pool.available() == pool.capacity
    e.cache.check()
    e.close()
    e, s = make(max_queue=1)
    r = e.submit([1, 2], 4)
    with pytest.raises(CapacityError):
        e.submit([1, 2], 4)
    r.events = queue.Queue(maxsize=1)
    drain(e)
    assert r.status == "error" and r.events.get()["finish_reason"] == "error"
    e.close()


def test_a_failing_step_ends_every_request_and_frees_everything():
    e, s = make()
    r = e.submit([1, 2], 3)
    s.fail = RuntimeError("test kernel failure")
    e.start()
    e.thread.join(timeout=3)
    assert "test kernel failure" in e.fatal
    assert r.events.get()["finish_reason"] == "error"
    assert len(e.cache.pools[0].free) == e.cache.pools[0].capacity
    with pytest.raises(RuntimeError):
        e.submit([1], 1)
    e.close()


def test_sampling_arguments_are_per_request():
    e, s = make()
    a = e.submit([1, 2, 3], 3, temperature=0.8, seed=9)
    b = e.submit([4, 5, 6, 7], 3)
    drain(e)
    temps, seeds, counters = e.sampler.last
    assert a.temperature == 0.8 and a.seed == 9 and b.temperature == 0.0
    assert len(a.output) == 3 and len(b.output) == 3
    e.close()


def test_generate_convenience_and_worker_thread():
    e, s = make()
    orig = e.submit
    prompts = [[1, 2, 3], [9, 8, 7, 6, 5, 4]]
    outs = e.generate(prompts, max_tokens=4)
    assert outs == [expected(p, 4) for p in prompts]
    r = orig([5, 5, 5], 3)
    e.start()
    got = []
    while True:
        ev = r.events.get(timeout=5)
        if ev["type"] == "done":
            break
        got.append(ev["token_id"])
    assert got == expected([5, 5, 5], 3) and e.stats()["finished"] == 3
    e.close()


# ---- lookahead: a turn is put on the device before the tokens of the turn before are read ----------
class FeedStepper(FakeStepper):
    """A step function that knows prompt tokens only; a negative id -1 - k is read from the token feed when
    the step runs, as the device does. Its logits come from the tokens IT has seen, not from the host's list."""
    accepts_token_feed = True
    token_feed = None

    def set_token_feed(self, feed):
        self.token_feed = feed

    def step(self, entries):
        rows = []
        self.batches.append([(e.seq.id, e.seq.computed, len(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            self.cache.ensure(e.seq, e.seq.computed + len(e.tokens))
            h = self.history.setdefault(e.seq.id, [])
            h.extend(self.full[e.seq.id][len(h):e.seq.computed])          # prefix-shared prompt tokens never ran here
            assert len(h) == e.seq.computed
            for t in e.tokens:
                assert t >= 0 or self.token_feed is not None
                h.append(t if t >= 0 else self.token_feed[-1 - t])
            self.fed += sum(t < 0 for t in e.tokens)
            for w in e.want:
                rows.append((e, e.seq.computed + w + 1))
        logits = torch.zeros(len(rows), VOCAB)
        for i, (e, upto) in enumerate(rows):
            logits[i, next_token(self.history[e.seq.id][:upto])] = 1.0
        for e in entries:
            self.cache.advance(e.seq, e.seq.computed + len(e.tokens))
        return logits

    fed = 0


class FeedSampler(FakeSampler):
    """Writes ids into one buffer that every call overwrites (the device's), hands back a copy later."""

    def __init__(self):
        self.out_buffer = [0] * 16
        self.unread = 0

    def sample_async(self, logits, temperatures, seeds, counters):
        ids = self.sample(logits, temperatures, seeds, counters)
        self.out_buffer[:len(ids)] = ids
        self.unread += 1
        sampler = self

        class Pending:
            def result(self):
                sampler.unread -= 1
                return list(ids)
        return Pending()


def make_lookahead(cfg=CFG, **kw):
    defaults = dict(block_size=4, kv_blocks=32, max_context=64, prefill_chunk=4, min_prefill_chunk=1, dtype="float32")
    defaults.update(kw)
    config = EngineConfig(**defaults)
    model = build_model(config_from_dict(cfg))
    cache = CacheManager(model.cache_layout(), config.block_size, config.kv_blocks, config.max_active,
                         prefix_cache=config.prefix_cache, max_request_tokens=config.max_context)
    stepper = FeedStepper(cache)
    stepper.full = {}
    engine = Engine(model, config, stepper=stepper, cache=cache, sampler=FeedSampler())
    submit = engine.submit

    def tracked(tokens, *a, **k):
        r = submit(tokens, *a, **k)
        stepper.full[r.id] = list(tokens)                              # the prompt only
        return r
    engine.submit = tracked
    return engine, stepper


def test_lookahead_gives_the_same_tokens_one_turn_late():
    e, s = make_lookahead()
    assert e.lookahead
    prompts = [[4, 5, 6, 7, 8], [2, 3, 4, 5, 6, 7, 8, 9, 10], [9]]
    counts = [7, 3, 1]
    rs = [e.submit(p, n) for p, n in zip(prompts, counts)]
    seen_unread = 0
    for _ in range(200):
        if not e.step():
            break
        seen_unread = max(seen_unread, e.sampler.unread)
        assert e.sampler.unread <= 1                                   # at most one turn's tokens are unread
    assert seen_unread == 1 and s.fed > 0                              # turns did run ahead of the host
    for r, p, n in zip(rs, prompts, counts):
        assert r.output == expected(p, n) and r.status == "length" and r.issued == n
    assert e._inflight is None and not e.requests
    e.cache.check()
    # no request ever ran past prompt + max_tokens - 1 positions
    for r, p, n in zip(rs, prompts, counts):
        assert len(s.history[r.id]) == len(p) + n - 1
    e.close()
    assert len(e.cache.pools[0].free) == 32
    # the same schedule of batches as without lookahead, apart from the reading
    e2, s2 = make(lookahead=False)
    for p, n in zip(prompts, counts):
        e2.submit(p, n)
    drain(e2)
    shape = lambda batches: [[(start, n, w) for _, start, n, w in b] for b in batches]
    assert shape(s.batches)[:3] == shape(s2.batches)[:3]
    e2.close()


def test_lookahead_drops_the_token_after_eos_and_frees_the_pages():
    prompt = [3, 4, 5, 6, 7]
    want = expected(prompt, 12)
    end = next(i for i in range(2, 12) if want[i] not in want[:i])
    e, s = make_lookahead(cfg=dict(CFG, eos_token_id=want[end]))
    r = e.submit(prompt, 12)
    other = e.submit([11, 12, 13], 12, ignore_eos=True)
    drain(e)
    assert r.status == "stop" and r.output == want[:end + 1]            # EOS is part of the output, nothing after it
    assert len(s.history[r.id]) == len(prompt) + end + 1               # ... though the device ran EOS's own step
    assert other.status == "length" and other.output == expected([11, 12, 13], 12)
    e.cache.check()
    e.close()
    assert len(e.cache.pools[0].free) == 32


def test_lookahead_with_cancel_failure_and_prefix_reuse():
    e, s = make_lookahead(prefix_cache=True)
    shared = list(range(1, 13))
    a = e.submit(shared + [20], 4)
    drain(e)
    b = e.submit(shared + [21], 4)                                      # 12 tokens = 3 pages come from the index
    c = e.submit([5, 6], 8)
    e.step(); e.step()
    e.cancel(c.id)                                                      # while one of its tokens is unread
    drain(e)
    assert b.cached == 12 and b.output == expected(shared + [21], 4) and a.output == expected(shared + [20], 4)
    assert c.status == "cancelled"
    e.cache.check()
    e.close()
    assert len(e.cache.pools[0].free) == 32


def test_a_prompt_portion_makes_room_for_decode_tokens_up_to_a_tile_of_rows():
    global CFG
    small, CFG = CFG, dict(CFG, max_position_embeddings=1024)
    try:
        _portion_and_tile_rows()
    finally:
        CFG = small


def _portion_and_tile_rows():
    e, s = make(kv_blocks=256, max_context=1024, prefill_chunk=256, min_prefill_chunk=16, max_active=4)
    short = [e.submit([1, 2, 3], 40) for _ in range(2)]
    e.step()                                                            # both short prompts complete, first tokens
    long = e.submit(list(range(100)) * 7, 4)                            # 700 tokens
    e.step()
    assert [(n, w) for _, _, n, w in s.batches[-1]] == [(1, [0]), (1, [0]), (254, [])]      # 2 + 254 = 256 rows, not 258
    e.step()
    assert [n for _, _, n, _ in s.batches[-1]] == [1, 1, 254]
    e.step()                                                            # 192 left: completes the prompt, never shortened
    assert [(n, w) for _, _, n, w in s.batches[-1]] == [(1, [0]), (1, [0]), (192, [191])]
    drain(e)
    assert long.output == expected(long.prompt, 4) and all(r.output == expected([1, 2, 3], 40) for r in short)
    e.close()
    e, s = make(kv_blocks=256, max_context=1024, prefill_chunk=256, min_prefill_chunk=16, max_active=4, tile_rows=0)
    a = e.submit([1, 2, 3], 40)
    e.step()
    e.submit(list(range(100)) * 7, 4)
    e.step()
    assert [n for _, _, n, _ in s.batches[-1]] == [1, 256]
    e.close()


@pytest.mark.parametrize("seed", range(6))
def test_random_arrivals_cancellations_and_both_ways_of_reading(seed):
    """Random prompts, budgets, arrival times and cancellations: with and without lookahead every request that
    is not cancelled gets the toy model's tokens, and no page is lost, held twice or left behind."""
    import random
    rng = random.Random(seed)
    plans = []
    for i in range(14):
        prompt = [rng.randrange(VOCAB) for _ in range(rng.choice([1, 2, 3, 5, 8, 13, 21, 30]))]
        plans.append(dict(prompt=prompt, max_tokens=rng.choice([1, 2, 3, 6, 11]), at=rng.randrange(0, 25),
                          cancel_at=rng.randrange(3, 40) if rng.random() < 0.25 else None,
                          temperature=rng.choice([0.0, 0.0, 0.7])))
    results = []
    for look in (True, False):
        make_engine = make_lookahead if look else make
        e, s = make_engine(kv_blocks=24, max_active=3, prefill_chunk=rng.choice([2, 4, 7]), prefix_cache=bool(seed % 2),
                           max_queue=32)
        assert e.lookahead == look
        live = {}
        for turn in range(400):
            for i, p in enumerate(plans):
                if p["at"] == turn:
                    live[i] = e.submit(p["prompt"], p["max_tokens"], temperature=p["temperature"], seed=i)
                if p["cancel_at"] == turn and i in live:
                    e.cancel(live[i].id)
            busy = e.step()
            e.cache.check()
            if not busy and turn > 45:
                break
        assert not e.requests and e._inflight is None
        out = {}
        for i, r in live.items():
            if r.status == "cancelled":
                assert r.output == expected(plans[i]["prompt"], len(r.output))       # a prefix of the right tokens
            else:
                assert r.status == "length" and r.output == expected(plans[i]["prompt"], plans[i]["max_tokens"])
            out[i] = (r.status, r.output if r.status != "cancelled" else None)
        e.close()
        assert len(e.cache.pools[0].free) == 24
        results.append(out)
    assert {i: v for i, v in results[0].items() if v[1] is not None and results[1][i][1] is not None} == \
           {i: v for i, v in results[1].items() if v[1] is not None and results[0][i][1] is not None}


def test_adaptive_portions_follow_the_measured_time_within_their_bounds():
    """The reference's feedback (flow_engine/engine.py:262-268): an EMA (0.8 / 0.2) of milliseconds per prompt
    token, the next portion = target / EMA, kept within [min_prefill_chunk, prefill_chunk]. Off by default."""
    e, s = make(prefill_chunk=64, min_prefill_chunk=4, target_step_ms=10.0, adaptive_chunk=True, max_context=128,
                kv_blocks=64)
    assert e.chunk == 64
    e._adapt_chunk(64.0, 64)                    # 1 ms a token: 10 tokens fit the target
    assert e.chunk == 10
    e._adapt_chunk(6.4, 64)                     # EMA 0.8 * 1 + 0.2 * 0.1 = 0.82
    assert e.chunk == 12
    for _ in range(60):
        e._adapt_chunk(0.64, 64)                # ever faster: capped at prefill_chunk
    assert e.chunk == 64
    for _ in range(60):
        e._adapt_chunk(6400.0, 64)              # ever slower: never below min_prefill_chunk
    assert e.chunk == 4
    # the next prompt portion has that size, and the prompt still completes
    r = e.submit(list(range(1, 40)), 3)
    e.step()
    assert s.batches[-1] == [(r.seq.id, 0, 4, [])]
    drain(e)
    assert r.output == expected(list(range(1, 40)), 3)
    e.close()
    fixed, s2 = make(prefill_chunk=8, min_prefill_chunk=1)
    r2 = fixed.submit(list(range(1, 30)), 2)
    drain(fixed)
    assert fixed.chunk == 8 and all(n <= 8 for batch in s2.batches for (_, _, n, _) in batch)
    fixed.close()


def test_generate_takes_more_tokens_than_an_event_queue_holds_and_seeds_each_prompt():
    cfg = dict(CFG, max_position_embeddings=1024)
    config = EngineConfig(block_size=4, kv_blocks=200, max_context=400, prefill_chunk=4, min_prefill_chunk=1,
                          dtype="float32")
    model = build_model(config_from_dict(cfg))
    cache = CacheManager(model.cache_layout(), 4, 200, config.max_active, max_request_tokens=400)
    stepper = FakeStepper(cache)
    stepper.full = {}
    e = Engine(model, config, stepper=stepper, cache=cache, sampler=FakeSampler())
    submit, made = e.submit, []

    def tracked(tokens, *a, **k):
        r = submit(tokens, *a, **k)
        stepper.full[r.id] = r.tokens
        made.append(r)
        return r
    e.submit = tracked
    outs = e.generate([[3, 1, 4], [3, 1, 4]], max_tokens=300, temperature=0.5, seed=40)
    assert [len(o) for o in outs] == [300, 300] and outs[0] == expected([3, 1, 4], 300)
    assert [r.seed for r in made] == [40, 41] and all(r.status == "length" for r in made)
    assert all(r.events.qsize() == 1 for r in made)                   # only the terminal event
    # a streaming consumer that never reads still loses its request after 256 tokens, as before
    r = tracked([3, 1, 4], 300)
    drain(e)
    assert r.status == "error" and len(r.output) == 257
    e.close()


def test_prompt_blocks_are_shared_while_their_first_owner_still_runs():
    e, s = make(max_active=2, prefill_chunk=8, max_step_tokens=8)
    prompt = [2, 3, 4, 5, 6, 7, 8, 9, 10]
    a = e.submit(prompt, 6)
    e.step()                                            # a's first 8 prompt tokens: two full blocks
    assert a.status == "active" and a.published == 8 and len(e.cache.pools[0].prefixes) == 2
    b = e.submit(prompt, 6)
    e.step()
    assert b.status == "active" and b.cached == 8 and a.status == "active"
    assert e.cache.stats()["prefix_hit_tokens"] == 8
    drain(e)
    assert a.output == b.output == expected(prompt, 6)
    # b never ran the shared tokens
    assert [(start, n) for batch in s.batches for (rid, start, n, _) in batch if rid == b.id][0] == (8, 1)
    e.close()
    e.cache.check()
    assert len(e.cache.pools[0].free) == 32


def test_a_head_of_queue_that_does_not_fit_earns_no_hits_and_costs_no_index_entries():
    e, s = make(kv_blocks=6, max_active=2)
    first = e.submit([1, 2, 3, 4, 5, 6, 7, 8, 9], 3)      # 3 pages
    drain(e)
    assert len(e.cache.pools[0].prefixes) == 2
    long_ = e.submit([7] * 9, 11)                         # 5 pages, admitted; evicts nothing yet needed
    e.step()
    entries = len(e.cache.pools[0].prefixes)
    again = e.submit([1, 2, 3, 4, 5, 6, 7, 8, 9], 3)      # shares 2 pages if they survived, needs 1 more: must wait
    waited = 0
    for _ in range(3):
        e.step()
        if again.status == "waiting":
            waited += 1
            assert e.cache.stats()["prefix_hit_tokens"] == 0
            assert len(e.cache.pools[0].prefixes) >= entries
    assert waited == 3
    drain(e)
    assert again.output == first.output and long_.status == "length"
    e.close()
    e.cache.check()


def test_prompt_blocks_are_shared_early_under_lookahead_too():
    e, s = make_lookahead(max_active=2, prefill_chunk=8, max_step_tokens=8)
    prompt = [2, 3, 4, 5, 6, 7, 8, 9, 10]
    a = e.submit(prompt, 6)
    e.step()
    b = e.submit(prompt, 6)
    e.step()
    assert b.status == "active" and b.cached == 8 and a.status == "active"
    drain(e)
    assert a.output == b.output == expected(prompt, 6)
    e.close()
    e.cache.check()
    assert len(e.cache.pools[0].free) == 32
