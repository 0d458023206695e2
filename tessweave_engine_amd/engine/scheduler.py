"""Continuous batching above the step function: admit, cut prompts, decode, finish, free.

Policy as the reference's engine (flow_engine/engine.py): FIFO admission with a
worst-case page reservation, so an admitted request can always finish and a
request that does not fit WAITS at the head of the queue (engine.py:96-113); a
request that could never fit is refused at submit (engine.py:81-82); every
turn decodes all ready requests and advances prompts round-robin
(engine.py:249-260); the portion that completes a prompt samples the first
token (engine.py:223-237); EOS is emitted and counted, then the request stops
(engine.py:169-174); pages are published to the prefix index on a normal finish
and released on any finish (engine.py:123-146).

Differences: the decode tokens and the prompt portions of a turn are ONE mixed
batch for the step function, under a token budget (`max_step_tokens`); several
prompts may advance in a turn if the budget allows; the portion size is fixed
unless `adaptive_chunk` asks for the reference's wall-clock feedback
(engine.py:262-268); sampling runs on the device.

Lookahead (`EngineConfig.lookahead`, on the GPU): a turn is put on the device
BEFORE the tokens of the turn before it are read. A request's newest token is then
named by its row in the sampler's output and resolved on the device, and the host
reads and commits tokens one turn late, while the device already runs the next
turn; the host's work between turns no longer leaves the device idle. A request
that turns out to have ended (EOS) has then run one token too far: that token is
dropped, and what it wrote lies beyond anything the prefix index publishes. The
tokens a request gets are the same with and without lookahead.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
import queue
import threading
import time
import uuid

from ..cache import CacheManager, CapacityError
from ..config import EngineConfig
from ..sampling.sampler import validate_temperature
from .step import StepEntry
from .trace import Trace

FINAL = ("stop", "length", "cancelled", "error")


@dataclass
class Request:
    id: str
    prompt: list
    max_tokens: int
    temperature: float
    seed: int
    namespace: str
    ignore_eos: bool = False
    tokens: list = field(default_factory=list)       # prompt + generated
    output: list = field(default_factory=list)       # generated
    seq: object = None                               # cache.Sequence while admitted
    issued: int = 0                                  # generated tokens, those still on the device included
    feed_row: int = -1                               # row of the newest token in the sampler's output while unread
    cached: int = 0                                  # prompt tokens taken from the prefix index
    status: str = "waiting"
    created: float = field(default_factory=time.perf_counter)
    first_token: float | None = None
    events: queue.Queue = field(default_factory=lambda: queue.Queue(maxsize=256))

    @property
    def computed(self):
        return self.seq.computed if self.seq is not None else 0

    @property
    def prefilling(self):
        return self.computed < len(self.prompt)


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
        self.counters = {"submitted": 0, "finished": 0, "cancelled": 0, "failed": 0,
                         "generated_tokens": 0, "prefill_tokens": 0, "steps": 0}

    # ---- requests in -------------------------------------------------------------------
    def submit(self, tokens, max_tokens=128, temperature=0.0, seed=0, namespace="local", ignore_eos=False):
        with self.lock:
            if self.fatal:
                raise RuntimeError(f"engine failed: {self.fatal}")
            vocab = self.model_config.vocab_size
            if not tokens or any(type(t) is not int or t < 0 or t >= vocab for t in tokens):
                raise ValueError("prompt must contain valid token ids")
            if type(max_tokens) is not int or max_tokens < 1 or len(tokens) + max_tokens > self.config.max_context:
                raise ValueError("prompt_tokens + max_tokens exceeds the configured context")
            temperature = validate_temperature(temperature)
            if not self.cache.fits(len(tokens) + max_tokens, self.config.step_token_budget):
                raise ValueError("this request alone exceeds the KV pool; increase --kv-blocks or reduce tokens")
            if len(self.waiting) >= self.config.max_queue:
                raise CapacityError("waiting queue is full")
            r = Request(uuid.uuid4().hex, list(tokens), max_tokens, temperature, int(seed), namespace, bool(ignore_eos))
            r.tokens = list(tokens)
            self.requests[r.id] = r
            self.waiting.append(r)
            self.counters["submitted"] += 1
            self.trace.emit("submit", request_id=r.id, prompt_tokens=len(tokens), max_tokens=max_tokens,
                            temperature=temperature, seed=seed)
            self.wake.set()
            return r

    def _admit(self):
        """FIFO: the head of the queue is admitted when a request slot and all its pages can be promised."""
        while self.waiting and len(self.active) < self.config.max_active:
            r = self.waiting[0]
            try:
                seq = self.cache.open(r.id)
            except CapacityError:
                break
            try:
                self.cache.acquire_prefix(seq, r.prompt, r.namespace)
                self.cache.reserve(seq, len(r.prompt) + r.max_tokens, self.config.step_token_budget)
            except CapacityError:
                self.cache.close(seq)
                break       # no skipping ahead: a large request is not starved by small ones
            self.waiting.popleft()
            r.seq, r.cached, r.status = seq, seq.cached, "active"
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
            logits = self.stepper.step(entries)
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

    def _sampling_stream(self):
        stream = getattr(self.stepper, "stream", None)
        if stream is None:
            import contextlib
            return contextlib.nullcontext()
        import torch
        return torch.cuda.stream(stream)

    def flush(self):
        """Read and commit the tokens of the last turn, if they are still unread (lookahead)."""
        with self.lock:
            self._collect()

    def _collect(self, turn=None):
        """Read the tokens a turn sampled (waiting for them if need be) and commit them to their requests."""
        if turn is None:
            turn, self._inflight = self._inflight, None
        if turn is None:
            return
        pending, rows = turn
        ids = pending.result() if hasattr(pending, "result") else pending
        for r, row in rows:
            if r.id in self.requests and r.status == "active":     # else it ended meanwhile: the token is dropped
                self._commit(r, int(ids[row]))

    def _adapt_chunk(self, elapsed_ms, prompt_tokens):
        # The reference's feedback (engine.py:262-268): EMA of prompt ms/token, portion sized to the turn budget.
        sample = elapsed_ms / max(1, prompt_tokens)
        self.prefill_ms_per_token = sample if self.prefill_ms_per_token is None else \
            .8 * self.prefill_ms_per_token + .2 * sample
        budget = max(1.0, self.config.target_step_ms)
        estimate = int(budget / max(.001, self.prefill_ms_per_token))
        self.chunk = max(self.config.min_prefill_chunk, min(self.config.prefill_chunk, estimate))

    # ---- tokens out, requests out -----------------------------------------------------
    def _emit(self, r, event):
        try:
            r.events.put_nowait(event)
            return True
        except queue.Full:
            self._finish(r, "error", "consumer too slow; bounded output queue exhausted")
            return False

    def _commit(self, r, token):
        r.tokens.append(token)
        r.output.append(token)
        self.counters["generated_tokens"] += 1
        if r.first_token is None:
            r.first_token = time.perf_counter()
            self.trace.emit("first_token", request_id=r.id, ttft_ms=(r.first_token - r.created) * 1000)
        if not self._emit(r, {"type": "token", "token_id": token}):
            return False
        if not r.ignore_eos and token in self.model_config.eos_token_ids:
            self._finish(r, "stop")
            return False
        if len(r.output) >= r.max_tokens:
            self._finish(r, "length")
            return False
        return True

    def _finish(self, r, reason, error=None):
        if r.id not in self.requests:
            return
        if r in self.active:
            if reason not in ("error", "cancelled"):
                self.cache.publish(r.seq, r.tokens, r.namespace)
            self.active.remove(r)
        elif r in self.waiting:
            self.waiting.remove(r)
        if r.seq is not None:
            self.cache.close(r.seq)
            r.seq = None
        r.status = reason
        del self.requests[r.id]
        self.counters[{"cancelled": "cancelled", "error": "failed"}.get(reason, "finished")] += 1
        end = {"type": "done", "finish_reason": reason, "error": error,
               "usage": {"prompt_tokens": len(r.prompt), "completion_tokens": len(r.output),
                         "total_tokens": len(r.prompt) + len(r.output)},
               "cached_tokens": r.cached, "elapsed_s": time.perf_counter() - r.created}
        if r.events.full():          # a terminal event always fits
            while not r.events.empty():
                r.events.get_nowait()
        r.events.put_nowait(end)
        self.trace.emit("finish", request_id=r.id, **{k: v for k, v in end.items() if k != "type"})

    def cancel(self, request_id):
        with self.lock:
            r = self.requests.get(request_id)
            if r:
                self._finish(r, "cancelled")

    # ---- worker thread -------------------------------------------------------------------
    def start(self):
        if self.running:
            return
        self.running = True
        self.thread = threading.Thread(target=self._loop, name="tessweave-model-worker", daemon=True)
        self.thread.start()

    def _loop(self):
        while self.running:
            try:
                if not self.step():
                    self.wake.wait(.05)
                    self.wake.clear()
            except Exception as exc:      # any failure of a step ends the engine, never a request silently
                self._fail(exc)
                self.running = False

    def _fail(self, exc):
        with self.lock:
            self.fatal = f"{type(exc).__name__}: {exc}"
            self.trace.emit("fatal", error=self.fatal)
            for r in list(self.requests.values()):
                self._finish(r, "error", self.fatal)

    def close(self):
        self.running = False
        self.wake.set()
        if self.thread:
            self.thread.join()           # storage is never freed while kernels are in flight
            self.thread = None
        with self.lock:
            for r in list(self.requests.values()):
                self._finish(r, "cancelled")
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
        """Token ids generated for each prompt (a list of id lists); runs on the calling thread."""
        requests, pending = [], list(prompts)
        while pending or self.requests:
            while pending and len(self.waiting) < self.config.max_queue:
                requests.append(self.submit(pending.pop(0), max_tokens, temperature, seed, ignore_eos=ignore_eos))
            if not self.step() and self.waiting:
                raise RuntimeError("a waiting request can never be admitted")
        failed = [r for r in requests if r.status == "error"]
        if failed:
            raise RuntimeError("generation failed")
        return [r.output for r in requests]

    def stats(self):
        with self.lock:
            return {**self.counters, **self.cache.stats(), "active": len(self.active),
                    "waiting": len(self.waiting), "prefill_chunk": self.chunk,
                    "ready": self.running and not self.fatal, "fatal": self.fatal,
                    "graph_replays": getattr(self.stepper, "graph_replays", 0)}
