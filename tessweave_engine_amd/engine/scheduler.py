"""Continuous batching above the step function: admit, cut prompts, decode, finish, free.

Policy as the reference's engine (flow_engine/engine.py): FIFO admission with a
worst-case page reservation, so an admitted request can always finish and a
request that does not fit WAITS at the head of the queue (engine.py:96-113); a
request that could never fit is refused at submit (engine.py:81-82); every
turn decodes all ready requests and advances prompts round-robin
(engine.py:249-260); the portion that completes a prompt samples the first
token (engine.py:223-237); EOS is emitted and counted, then the request stops
(engine.py:169-174); pages are published to the prefix index on a normal finish
and released on any finish (engine.py:123-146); a consumer that lets its bounded
event queue fill up loses the request, never the engine (engine.py:115-121).

Differences: the decode tokens and the prompt portions of a turn are ONE mixed
batch for the step function, under a token budget (`max_step_tokens`); several
prompts may advance in a turn if the budget allows; the portion size is fixed
unless `adaptive_chunk` asks for the reference's wall-clock feedback
(engine.py:262-268); sampling runs on the device; the full blocks of a prompt
are entered into the prefix index as soon as the step that computes them has
been issued, so requests that are live at the same time share them (the
reference shares only what a finished request leaves, engine.py:127-128).

Lookahead (`EngineConfig.lookahead`, on the GPU): a turn is put on the device
BEFORE the tokens of the turn before it are read. A request's newest token is then
named by its row in the sampler's output and resolved on the device, and the host
reads and commits tokens one turn late, while the device already runs the next
turn; the host's work between turns no longer leaves the device idle. A request
that turns out to have ended (EOS) has then run one token too far: that token is
dropped, and what it wrote lies beyond anything the prefix index publishes.
With and without lookahead a request's logits are the same up to rounding: in
32-bit its tokens are the same; in bfloat16 a choice between two words whose
logits lie within bfloat16's rounding of each other (or a draw that falls on
the edge between two words) may go either way, because lookahead retires a
request one turn later, so the same token can meet another batch (beside a
prompt portion it runs through the tiled kernels, alone through the streaming
ones, which sum in another order). The same holds for any two schedules.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass
import contextlib
import queue
import threading
import time
import uuid

from ..cache import CacheManager, CapacityError
from ..config import EngineConfig
from ..sampling.sampler import validate_temperature
from .step import StepEntry
from .trace import Trace

#: a request's status is "waiting", "active" or the reason it ended
ENDED_NORMALLY = ("stop", "length")
ENDED = ENDED_NORMALLY + ("cancelled", "error")
EVENT_QUEUE_DEPTH = 256          # flow_engine/engine.py:32


class Request:
    """One generation request, from `submit` to its terminal event.

    `events` carries {"type": "token", "token_id": t} for every generated token and one final
    {"type": "done", ...}. It is bounded; a request made with stream=False has no token events (its
    tokens are read from `output` once it has ended) and can therefore not overrun the queue.
    """

    def __init__(self, prompt, max_tokens, temperature, seed, namespace, ignore_eos, stream=True):
        self.id = uuid.uuid4().hex
        self.prompt = list(prompt)
        self.max_tokens = max_tokens
        self.temperature = temperature
        self.seed = int(seed)
        self.namespace = namespace
        self.ignore_eos = bool(ignore_eos)
        self.stream = bool(stream)
        self.tokens = list(prompt)      # prompt + generated
        self.output = []                # generated
        self.seq = None                 # cache.Sequence while admitted
        self.issued = 0                 # generated tokens, those still on the device included
        self.feed_row = -1              # row of the newest token in the sampler's output while unread
        self.cached = 0                 # prompt tokens taken from the prefix index
        self.published = 0              # prompt tokens whose full blocks were offered to the prefix index
        self.status = "waiting"
        self.created = time.perf_counter()
        self.first_token = None
        self.events = queue.Queue(maxsize=EVENT_QUEUE_DEPTH)

    @property
    def computed(self):
        return self.seq.computed if self.seq is not None else 0

    @property
    def prefilling(self):
        return self.computed < len(self.prompt)

    @property
    def ended(self):
        return self.status in ENDED

    def usage(self):
        n_in, n_out = len(self.prompt), len(self.output)
        return {"prompt_tokens": n_in, "completion_tokens": n_out, "total_tokens": n_in + n_out}


@dataclass
class Portion:
    request: Request
    count: int                    # tokens of the request in this step
    samples: bool                 # the step's last token of this request yields a new token
    prompt: bool = False          # the tokens are part of the prompt


class Engine:
    def __init__(self, model, config=None, trace=None, *, stepper=None, cache=None, sampler=None):
        """MODEL gives `.config` and `.cache_layout()`; STEPPER, CACHE, SAMPLER default to the GPU ones."""
        self.model = model
        self.model_config = model.config
        self.config = config or EngineConfig()
        if self.config.max_context > self.model_config.max_position_embeddings:
            raise ValueError("requested context exceeds the model's max_position_embeddings")
        self.cache = cache or CacheManager(
            model.cache_layout(), self.config.block_size, self.config.kv_blocks, self.config.max_active,
            dtype=self.config.dtype, device=model.device, prefix_cache=self.config.prefix_cache,
            max_request_tokens=self.config.max_context)
        if stepper is None:
            from .step import Stepper
            stepper = Stepper(model, self.cache, max_step_tokens=self.config.step_token_budget,
                              max_step_seqs=self.config.max_active, use_graphs=self.config.use_graphs)
        self.stepper = stepper
        if sampler is None:
            from ..sampling.sampler import DeviceSampler
            sampler = DeviceSampler(model.device, self.config.max_active)
        self.sampler = sampler
        self.trace = trace or Trace()
        self.waiting = deque()
        self.active = []
        self.requests = {}
        self.lock = threading.RLock()
        self.wake = threading.Event()
        self.running = False
        self.thread = None
        self.fatal = None
        self.lookahead = (bool(getattr(self.config, "lookahead", True)) and hasattr(self.sampler, "sample_async")
                          and getattr(self.stepper, "accepts_token_feed", False))
        self._inflight = None            # (PendingTokens, [(request, row)]) of the turn whose tokens are unread
        self.prefill_cursor = 0
        self.chunk = self.config.prefill_chunk
        self.prefill_ms_per_token = None
        self.counters = dict.fromkeys(("submitted", "finished", "cancelled", "failed", "generated_tokens",
                                       "prefill_tokens", "steps"), 0)

    # ---- requests in -------------------------------------------------------------------
    def _refuse_unless_valid(self, tokens, max_tokens):
        """What `submit` refuses for good (flow_engine/engine.py:75-82): ids outside the vocabulary, a
        budget beyond the configured context, a request that the whole cache could not hold."""
        vocab = self.model_config.vocab_size
        if len(tokens) == 0:
            raise ValueError("an empty prompt cannot be run")
        for t in tokens:
            if type(t) is not int or not 0 <= t < vocab:
                raise ValueError(f"prompt token {t!r} is no id in [0, {vocab})")
        if type(max_tokens) is not int or max_tokens < 1:
            raise ValueError("max_tokens must be a positive integer")
        total = len(tokens) + max_tokens
        if total > self.config.max_context:
            raise ValueError(f"prompt ({len(tokens)}) + max_tokens ({max_tokens}) exceeds the configured "
                             f"context of {self.config.max_context}")
        if not self.cache.fits(total, self.config.step_token_budget):
            raise ValueError(f"{total} tokens need more pages than the cache has; raise --kv-blocks or ask for fewer")

    def submit(self, tokens, max_tokens=128, temperature=0.0, seed=0, namespace="local", ignore_eos=False,
               stream=True):
        """Queue a request; returns its `Request`. ValueError: it can never run. CapacityError: the queue is full."""
        with self.lock:
            if self.fatal:
                raise RuntimeError(f"engine failed: {self.fatal}")
            self._refuse_unless_valid(tokens, max_tokens)
            temperature = validate_temperature(temperature)
            if len(self.waiting) >= self.config.max_queue:
                raise CapacityError("waiting queue is full")
            r = Request(tokens, max_tokens, temperature, seed, namespace, ignore_eos, stream)
            self.requests[r.id] = r
            self.waiting.append(r)
            self.counters["submitted"] += 1
            self.trace.emit("submit", request_id=r.id, prompt_tokens=len(r.prompt), max_tokens=max_tokens,
                            temperature=temperature, seed=r.seed)
        self.wake.set()
        return r

    def _admit(self):
        """Admit from the head of the queue while a request slot and every page the head can ever need are
        to be had. A head that does not fit stops admission: nobody overtakes it, so it cannot starve."""
        budget = self.config.step_token_budget
        while self.waiting and len(self.active) < self.config.max_active:
            r = self.waiting[0]
            try:
                r.seq = self.cache.admit(r.id, r.prompt, len(r.prompt) + r.max_tokens, budget, r.namespace)
            except CapacityError:
                return
            self.waiting.popleft()
            r.cached = r.published = r.seq.cached
            r.status = "active"
            self.active.append(r)
            self.trace.emit("admit", request_id=r.id, reused_tokens=r.cached, **self.cache.stats())

    # ---- one turn ----------------------------------------------------------------------
    def plan(self):
        """Which admitted requests run how many tokens in the next step (decisions only, no side effects
        beyond the round-robin cursor)."""
        decode = [r for r in self.active if not r.prefilling and r.issued < r.max_tokens]
        portions = [Portion(r, 1, True) for r in decode]
        prefill = [r for r in self.active if r.prefilling]
        if prefill:
            budget = self.config.step_token_budget - len(decode)
            start = self.prefill_cursor % len(prefill)
            self.prefill_cursor += 1
            for i in range(len(prefill)):
                r = prefill[(start + i) % len(prefill)]
                remaining = len(r.prompt) - r.computed
                count = min(self.chunk, remaining, budget)
                if count < 1:
                    break
                # After the first portion, no crumbs: a further prompt advances only by a useful amount.
                if i > 0 and count < min(self.config.min_prefill_chunk, remaining):
                    break
                portions.append(Portion(r, count, count == remaining, True))
                budget -= count
            # The matrix kernels work on tiles of 128 rows: a step of 256 prompt tokens and 8 decode
            # tokens would pay for 384. If the decode tokens alone push the step past a multiple of the
            # tile, the last portion gives up that many tokens (unless it completes its prompt).
            tile = self.config.tile_rows
            last = portions[-1]
            if tile and last.prompt and not last.samples:
                excess = (len(decode) + sum(p.count for p in portions if p.prompt)) % tile
                if 0 < excess <= len(decode) and last.count - excess >= self.config.min_prefill_chunk:
                    last.count -= excess
        return portions

    def step(self):
        """One scheduler turn; False when nothing is admitted and no token is unread."""
        with self.lock:
            self._admit()
            portions = self.plan() if self.active else []
            if not portions:
                if self._inflight is None:
                    return False
                self._collect()              # nothing new to run: read what the last turn sampled
                return True
            started = time.perf_counter()
            if self.lookahead:
                feed = self.sampler.out_buffer
                if getattr(self.stepper, "token_feed", None) is not feed:
                    self.stepper.segment_graphs = False      # launches are hidden behind the step before
                    self.stepper.set_token_feed(feed)
            entries = []
            for p in portions:
                r = p.request
                begin = r.computed
                if begin == len(r.tokens):   # its newest token is still on the device: name it by its row
                    tokens = [-1 - r.feed_row]
                else:
                    tokens = r.tokens[begin:begin + p.count]
                entries.append(StepEntry(r.seq, tokens, [p.count - 1] if p.samples else []))
            # (everything of a turn is issued on the step's own stream: nothing waits for another stream)
            with self._sampling_stream():
                logits = self.stepper.step(entries)
            self._publish_prompt_blocks(portions)
            sampled = [p for p in portions if p.samples]
            arguments = (logits, [p.request.temperature for p in sampled], [p.request.seed for p in sampled],
                         [p.request.issued for p in sampled])
            previous = self._inflight
            if not sampled:
                self._inflight = None
            elif self.lookahead:
                # on the step's own stream: the sampling kernels follow the step without a wait between streams
                with self._sampling_stream():
                    pending = self.sampler.sample_async(*arguments)
                self._inflight = (pending, [(p.request, i) for i, p in enumerate(sampled)])
            else:
                with self._sampling_stream():
                    ids = self.sampler.sample(*arguments)
                self._inflight = (ids, [(p.request, i) for i, p in enumerate(sampled)])
            for i, p in enumerate(sampled):
                p.request.issued += 1
                p.request.feed_row = i
            if previous is not None:
                self._collect(previous)      # the turn before, read while the device runs this one
            if not self.lookahead:
                self._collect()
            elif not sampled and self.config.adaptive_chunk and hasattr(self.stepper, "synchronize"):
                self.stepper.synchronize()      # nothing was read back: wait so that the timing is real
            elapsed = (time.perf_counter() - started) * 1000
            self.counters["steps"] += 1
            n_prompt = sum(p.count for p in portions if p.prompt)
            self.counters["prefill_tokens"] += n_prompt
            self.trace.emit("step", request_ids=[p.request.id for p in portions], batch=len(portions),
                            tokens=sum(p.count for p in portions), prompt_tokens=n_prompt,
                            elapsed_ms=elapsed, prefill_chunk=self.chunk, **self.cache.stats())
            if self.config.adaptive_chunk and n_prompt:
                self._adapt_chunk(elapsed, n_prompt)
            return True

    def _publish_prompt_blocks(self, portions):
        """Offer the prompt blocks that the step just issued completes to the prefix index.

        Safe before the step has finished: whoever takes such a page reads it in a later step, and all
        device work is ordered on one stream; the owner itself writes only beyond its computed length, so
        a published page is never written again.
        """
        if not self.cache.prefix_cache:
            return
        page = self.cache.page_size
        for p in portions:
            r = p.request
            if not p.prompt or r.seq is None or r.seq.closed:
                continue
            whole = min(r.computed, len(r.prompt)) // page * page
            if whole > r.published:
                self.cache.publish(r.seq, r.prompt, r.namespace, computed=whole)    # hashes only the new blocks
                r.published = whole

    def _sampling_stream(self):
        stream = getattr(self.stepper, "stream", None)
        if stream is None:
            return contextlib.nullcontext()
        import torch
        return torch.cuda.stream(stream)

    def flush(self):
        """Read and commit the tokens of the last turn, if they are still unread (lookahead)."""
        with self.lock:
            self._collect()

    def _collect(self, turn=None):
        """Read the tokens a turn sampled (waiting for them if need be) and hand them to their requests."""
        if turn is None:
            turn, self._inflight = self._inflight, None
        if turn is None:
            return
        pending, rows = turn
        ids = pending.result() if hasattr(pending, "result") else pending
        for r, row in rows:
            if r.status == "active":         # else it ended meanwhile: the token is dropped
                self._accept(r, int(ids[row]))

    def _adapt_chunk(self, elapsed_ms, prompt_tokens):
        # The reference's feedback (engine.py:262-268): EMA of prompt ms/token, portion sized to the turn budget.
        sample = elapsed_ms / max(1, prompt_tokens)
        self.prefill_ms_per_token = sample if self.prefill_ms_per_token is None else \
            .8 * self.prefill_ms_per_token + .2 * sample
        budget = max(1.0, self.config.target_step_ms)
        estimate = int(budget / max(.001, self.prefill_ms_per_token))
        self.chunk = max(self.config.min_prefill_chunk, min(self.config.prefill_chunk, estimate))

    # ---- tokens out, requests out -----------------------------------------------------
    def _accept(self, r, token):
        """A sampled token reaches its request: record it, tell the consumer, and end the request if this
        token is an EOS (it is still delivered and counted) or the last one asked for."""
        now = time.perf_counter()
        r.tokens.append(token)
        r.output.append(token)
        self.counters["generated_tokens"] += 1
        if r.first_token is None:
            r.first_token = now
            self.trace.emit("first_token", request_id=r.id, ttft_ms=(now - r.created) * 1000)
        if r.stream:
            try:
                r.events.put_nowait({"type": "token", "token_id": token})
            except queue.Full:
                self._retire(r, "error", "consumer too slow; bounded output queue exhausted")
                return
        if token in self.model_config.eos_token_ids and not r.ignore_eos:
            self._retire(r, "stop")
        elif len(r.output) >= r.max_tokens:
            self._retire(r, "length")

    def _retire(self, r, reason, error=None):
        """The one place a request ends, for any reason: out of the engine's lists, cache given back (its
        full blocks published first if it ended normally), counters, and the terminal event, which always
        fits: a consumer that stopped reading loses its unread tokens, not the verdict."""
        if r.ended:
            return
        was, r.status = r.status, reason
        self.requests.pop(r.id, None)
        if was == "waiting":
            self.waiting.remove(r)
        else:
            self.active.remove(r)
        if r.seq is not None:
            if reason in ENDED_NORMALLY:
                self.cache.publish(r.seq, r.tokens, r.namespace)
            self.cache.close(r.seq)
            r.seq = None
        tally = "finished" if reason in ENDED_NORMALLY else "cancelled" if reason == "cancelled" else "failed"
        self.counters[tally] += 1
        verdict = {"finish_reason": reason, "error": error, "usage": r.usage(), "cached_tokens": r.cached,
                   "elapsed_s": time.perf_counter() - r.created}
        while True:
            try:
                r.events.put_nowait({"type": "done", **verdict})
                break
            except queue.Full:
                with contextlib.suppress(queue.Empty):
                    r.events.get_nowait()
        self.trace.emit("finish", request_id=r.id, **verdict)

    def cancel(self, request_id):
        """End a waiting or running request now; unknown and ended ids are ignored."""
        with self.lock:
            r = self.requests.get(request_id)
            if r is not None:
                self._retire(r, "cancelled")

    # ---- worker thread -------------------------------------------------------------------
    def start(self):
        """Run turns on a worker thread until `close`; the thread sleeps while there is nothing to do."""
        if self.running:
            return
        self.running = True
        self.thread = threading.Thread(target=self._work, name="tessweave-model-worker", daemon=True)
        self.thread.start()

    def _work(self):
        try:
            while self.running:
                if not self.step():
                    self.wake.wait(0.05)
                    self.wake.clear()
        except Exception as exc:          # a failing step ends the engine and tells every request; none is lost silently
            self._fail(exc)
        finally:
            self.running = False

    def _fail(self, exc):
        with self.lock:
            self.fatal = f"{type(exc).__name__}: {exc}"
            self.trace.emit("fatal", error=self.fatal)
            for r in list(self.requests.values()):
                self._retire(r, "error", self.fatal)

    def close(self):
        """Stop the worker (waiting for the step it is in: storage is never freed under running kernels),
        cancel what is left, empty the prefix index and drop the captured graphs."""
        self.running = False
        self.wake.set()
        thread, self.thread = self.thread, None
        if thread is not None:
            thread.join()
        with self.lock:
            for r in list(self.requests.values()):
                self._retire(r, "cancelled")
            self.cache.clear_prefixes()
            if hasattr(self.stepper, "close"):
                self.stepper.close()
        self.trace.close()

    def drain(self, max_steps=1_000_000):
        """Run turns on the calling thread until nothing is admitted or waiting."""
        for _ in range(max_steps):
            if not self.step():
                return
        raise RuntimeError("engine did not finish")

    def generate(self, prompts, max_tokens=128, temperature=0.0, seed=0, ignore_eos=False):
        """Token ids generated for each prompt (a list of id lists); runs on the calling thread.

        Prompt i samples with seed SEED + i, so equal prompts do not draw equal streams. The requests
        have no token events, so any `max_tokens` is fine.
        """
        prompts = list(prompts)
        requests = []
        while len(requests) < len(prompts) or self.requests:
            while len(requests) < len(prompts) and len(self.waiting) < self.config.max_queue:
                i = len(requests)
                requests.append(self.submit(prompts[i], max_tokens, temperature, seed + i, ignore_eos=ignore_eos,
                                            stream=False))
            if not self.step() and self.waiting:
                raise RuntimeError("a waiting request can never be admitted")
        for r in requests:
            if r.status == "error":
                raise RuntimeError(f"generation failed: {r.events.get_nowait().get('error')}")
        return [r.output for r in requests]

    def stats(self):
        with self.lock:
            return {**self.counters, **self.cache.stats(), "active": len(self.active),
                    "waiting": len(self.waiting), "prefill_chunk": self.chunk,
                    "ready": self.running and not self.fatal, "fatal": self.fatal,
                    "graph_replays": getattr(self.stepper, "graph_replays", 0)}
