"""The step function: one batch of (request, its next tokens) through the model, from the cache.

The reference runs two uniform forwards per scheduler turn, a [B,1] decode
batch and then one [1,T] prompt portion (flow_engine/engine.py:249-260,
model.py:169), and rebuilds and uploads slot lists per layer
(model.py:178, cache.py:98,105-107). Here one call takes any mix of prompt
portions and single decode tokens as ONE flat batch: the metadata of the step
(token ids, positions, cache slots, block tables, lengths, wanted rows) is
packed on the host into a single int32 buffer, uploaded once, and every layer
only reads it. Logits come back in float32 for exactly the rows asked for.

Decode-only steps of a model whose parts are all graph-safe are captured once
per (batch size, length class) into a HIP graph and replayed; only the metadata
upload differs between replays. The length class is the longest sequence of
the step rounded up to a power of two: launch shapes that should follow the
lengths (the number of key ranges of decode attention) follow the class, so an
engine opened for 32,768 tokens that serves 2,000-token requests runs the
launches of a 2,048-token engine.
"""
from __future__ import annotations

from collections import OrderedDict
import ctypes
from dataclasses import dataclass, field

import numpy as np
import torch

from ..kernels import ops
from ..kernels.lib import library, check
from ..parts.base import GroupStep, StepContext, Workspace


@dataclass
class StepEntry:
    seq: object                      # cache.Sequence
    tokens: list                     # the request's next tokens (at least one)
    want: list = field(default_factory=list)   # indices into tokens whose logits are wanted
    positions: object = None         # None: every position axis counts the request's tokens (computed, computed + 1, ...);
                                     # else one list of len(tokens) position ids per axis of the model's encodings.
                                     # The cache and the causal order go by token order, whatever the ids say.


def _round_up(v, m):
    return (v + m - 1) // m * m


GRAPH_SEGMENT_RUNS = 8       # layer runs per captured graph after the first
MIN_LENGTH_CLASS = 512       # steps whose longest sequence is shorter share one captured graph
MAX_GRAPHS = 96              # captured steps kept (one per batch size and length class met); the least recently
                             # replayed one goes first


class _Graph:
    """A captured decode step: several graphs launched one after the other (see Stepper._capture).

    BUFFERS names the scratch buffers whose addresses the capture holds, each with its version at the
    time: the capture stays good until one of THOSE is allocated anew (a larger prompt portion growing a
    buffer that only prompt portions use leaves every captured decode step alone)."""

    def __init__(self, handles, logits, generation, buffers):
        self.handles, self.logits, self.generation, self.buffers = handles, logits, generation, buffers


class Stepper:
    def __init__(self, model, cache, max_step_tokens=256, max_step_seqs=None, use_graphs=True, max_graphs=MAX_GRAPHS):
        if model.device is None or model.device.type != "cuda":
            raise RuntimeError("the model's weights must be on a GPU: there is no CPU path")
        self.model = model
        self.cache = cache
        self.device = model.device
        self.dtype = model.dtype
        self.workspace = Workspace(self.device)
        self.stream = torch.cuda.Stream(device=self.device)
        self.use_graphs = bool(use_graphs) and model.graph_safe_model
        self._defer_sums = bool(getattr(model, "defers_sums", False))
        self.position_axes = max(1, int(getattr(model, "position_axes", 1)))
        self.max_tokens = 0
        self.max_seqs = 0
        self._graphs = OrderedDict()     # (batch size, length class) -> _Graph, least recently replayed first
        self._warm = set()
        self.max_graphs = max(1, int(max_graphs))
        self.token_feed = None
        self.segment_graphs = True
        self._staging = []
        self._staging_events = []
        self._staging_next = 0
        self.steps = 0
        self.graph_replays = 0
        self._reserve(max(1, int(max_step_tokens)), int(max_step_seqs or cache.max_requests))

    # ---- metadata buffers ------------------------------------------------------------
    def _reserve(self, max_tokens, max_seqs):
        """(Re)allocate the metadata buffers for steps of up to MAX_TOKENS rows and MAX_SEQS requests."""
        self._drop_graphs()
        self.max_tokens, self.max_seqs = max_tokens, max_seqs
        width = self.cache.table_width
        n_groups = len(self.cache.pools)
        sections, offset = {}, 0

        def add(name, count):
            nonlocal offset
            sections[name] = (offset, count)
            offset += _round_up(count, 64)

        add("token_ids", max_tokens)
        add("positions", self.position_axes * max_tokens)
        add("q_start", max_seqs + 1)
        add("kv_len", max_seqs)
        add("state_slots", max_seqs)
        add("logit_rows", max_tokens)
        for g in range(n_groups):
            add(f"slots{g}", max_tokens)
            add(f"table{g}", max_seqs * width)
        self._sections, self._meta_ints = sections, offset
        self._meta_dev = torch.zeros(offset, dtype=torch.int32, device=self.device)
        self._staging = [torch.zeros(offset, dtype=torch.int32, pin_memory=True) for _ in range(4)]
        self._staging_np = [t.numpy() for t in self._staging]
        self._staging_events = [None] * 4
        self._staging_next = 0

    def _dev(self, name, count=None):
        off, cap = self._sections[name]
        return self._meta_dev[off:off + (cap if count is None else count)]

    def _drop_graphs(self):
        if self._graphs:
            torch.cuda.synchronize(self.device)
            lib = library()
            for graph in self._graphs.values():
                for handle in graph.handles:
                    lib.tw_graph_destroy(handle)
        self._graphs = OrderedDict()
        self._warm = set()

    def _drop_graph(self, key):
        """Destroy one captured step (it may still be running: wait for the step's stream first)."""
        graph = self._graphs.pop(key)
        self.stream.synchronize()
        lib = library()
        for handle in graph.handles:
            lib.tw_graph_destroy(handle)

    def close(self):
        self._drop_graphs()

    accepts_token_feed = True

    def set_token_feed(self, feed):
        """FEED (int32, on the device, or None): from now on a token id -1 - k in a step entry stands for
        feed[k] as it is when the step runs, e.g. a token sampled by the step before that the host has not read."""
        if feed is not None and (feed.dtype != torch.int32 or feed.device.type != "cuda" or not feed.is_contiguous()):
            raise ValueError("the token feed must be a contiguous int32 tensor on the model's device")
        same = (feed is None and self.token_feed is None) or \
            (feed is not None and self.token_feed is not None and feed.data_ptr() == self.token_feed.data_ptr()
             and feed.numel() == self.token_feed.numel())
        if not same:
            self._drop_graphs()          # captured steps hold the old pointer
            self.token_feed = feed

    def synchronize(self):
        self.stream.synchronize()

    # ---- the step ----------------------------------------------------------------------
    def step(self, entries):
        """Run ENTRIES as one batch; float32 logits [sum(len(e.want)), vocab] in the order of entries and want.

        The returned tensor is scratch memory: read or copy it before the next step.
        """
        entries = list(entries)
        if not entries:
            return torch.empty(0, self.model.vocab_size, dtype=torch.float32, device=self.device)
        ctx, ordered, graphable = self.prepare(entries)
        # A caller that already works on the step's stream (the scheduler with lookahead) needs no hand-over
        # between streams. Each hand-over is an event and a wait in another hardware queue, unless the two
        # streams happen to share a queue (one engine in four of a process did, and ran 0.2 ms a step faster).
        caller = torch.cuda.current_stream(self.device)
        same = caller.cuda_stream == self.stream.cuda_stream
        if not same:
            self.stream.wait_stream(caller)
        with torch.cuda.stream(self.stream):
            self.upload(ctx)
            if graphable:
                logits = self._run_graphable(ctx, (ctx.n_seqs, ctx.kv_bound))
            else:
                logits = self.model.forward(ctx)
        if not same:
            caller.wait_stream(self.stream)
        self.finish(ordered)
        return logits

    def finish(self, ordered):
        """Record in the cache that the step's tokens are now held."""
        for e in ordered:
            self.cache.advance(e.seq, e.seq.computed + len(e.tokens))
        self.steps += 1

    def upload(self, ctx):
        """Bring the step's packed metadata to the device (on the current stream): a kernel fetches the parts
        this step filled from the pinned staging buffer, which keeps the step in one queue (a memory copy
        would hand over to the copy engine and back, tens of microseconds of idle queue per step)."""
        k = ctx.staging_index
        if ctx.staging_segments is not None and len(ctx.staging_segments) <= 16:
            ops.upload_words(self._staging[k], self._meta_dev, ctx.staging_segments)
        else:
            self._meta_dev.copy_(self._staging[k], non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        self._staging_events[k] = event

    def prepare(self, entries):
        """Check ENTRIES, take their pages, and build the step's context (host side; nothing runs yet).

        Returns (context, entries in batch order, whether the step can be replayed from a graph).
        """
        vocab, seen = self.model.vocab_size, set()
        feed = self.token_feed.numel() if self.token_feed is not None else 0     # ids -1 .. -feed name fed tokens
        for e in entries:
            if not e.tokens:
                raise ValueError("a step entry needs at least one token")
            if id(e.seq) in seen:
                raise ValueError("a request appears twice in one step")
            seen.add(id(e.seq))
            if e.seq.closed:
                raise ValueError(f"request {e.seq.id!r} is closed")
            if any(type(t) is not int or t >= vocab or t < -feed for t in e.tokens):
                raise ValueError(f"request {e.seq.id!r}: token ids must be integers in [0, {vocab})")
            if any(type(w) is not int or w < 0 or w >= len(e.tokens) for w in e.want):
                raise ValueError(f"request {e.seq.id!r}: wanted places must index this step's tokens")
            if e.positions is not None and (len(e.positions) != self.position_axes
                                            or any(len(axis) != len(e.tokens) for axis in e.positions)):
                raise ValueError(f"request {e.seq.id!r}: positions must be {self.position_axes} lists of one id per token")
        n_tokens = sum(len(e.tokens) for e in entries)
        if n_tokens > self.max_tokens or len(entries) > self.max_seqs:
            self._reserve(max(self.max_tokens, _round_up(n_tokens, 256)), max(self.max_seqs, len(entries)))
        for e in entries:
            self.cache.ensure(e.seq, e.seq.computed + len(e.tokens))

        # decode entries (one token) first, then prompt portions; stable
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) != 1)
        ordered = [entries[i] for i in order]
        n_seqs = len(ordered)
        q_lens = np.fromiter((len(e.tokens) for e in ordered), dtype=np.int64, count=n_seqs)
        n_decode = int((q_lens == 1).sum())
        computed = np.fromiter((e.seq.computed for e in ordered), dtype=np.int64, count=n_seqs)
        slots_of = np.fromiter((e.seq.state_slot for e in ordered), dtype=np.int64, count=n_seqs)
        q_start = np.zeros(n_seqs + 1, dtype=np.int64)
        np.cumsum(q_lens, out=q_start[1:])
        kv_len = computed + q_lens
        seq_of_token = np.repeat(np.arange(n_seqs), q_lens)
        positions = np.arange(n_tokens) - np.repeat(q_start[:-1] - computed, q_lens)
        if n_decode == n_seqs:
            token_ids = np.fromiter((e.tokens[0] for e in ordered), dtype=np.int64, count=n_seqs)
        else:
            token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in ordered])
        position_in_order = {orig: pos for pos, orig in enumerate(order)}
        rows = [int(q_start[position_in_order[i]]) + w for i, e in enumerate(entries) for w in e.want]
        n_logits = len(rows)

        # pack the metadata into a pinned buffer and upload it once
        k = self._staging_next
        self._staging_next = (k + 1) % len(self._staging)
        if self._staging_events[k] is not None:
            self._staging_events[k].synchronize()
        host = self._staging_np[k]

        segments = []                        # (offset, words) of what this step fills: all that has to travel

        def put(name, values):
            off, _ = self._sections[name]
            host[off:off + len(values)] = values
            segments.append((off, len(values)))

        put("token_ids", token_ids)
        axes = self.position_axes
        ids = np.tile(positions, (axes, 1))                      # [axes, n_tokens]; `positions` stays the token order
        for s_index, e in enumerate(ordered):
            if e.positions is not None:
                ids[:, q_start[s_index]:q_start[s_index + 1]] = np.asarray(e.positions, dtype=np.int64)
        put("positions", ids.reshape(-1))
        put("q_start", q_start)
        put("kv_len", kv_len)
        put("state_slots", slots_of)
        put("logit_rows", np.asarray(rows, dtype=np.int64))
        page = self.cache.page_size
        width = self.cache.table_width
        for g in range(len(self.cache.pools)):
            tables = self.cache.table_rows[g][slots_of]                       # [n_seqs, width]
            pages = tables[seq_of_token, positions // page]
            first = self._first_positions(g, computed)
            live = positions >= np.repeat(first, q_lens)
            if (pages[live] < 0).any():
                raise RuntimeError("a token's page is not held; the cache manager and the step disagree")
            put(f"slots{g}", np.where(pages >= 0, pages * page + positions % page, -1))
            off, _ = self._sections[f"table{g}"]
            host[off:off + n_seqs * width] = tables.reshape(-1)
            segments.append((off, n_seqs * width))

        ctx = StepContext()
        ctx.device, ctx.dtype = self.device, self.dtype
        ctx.n_tokens, ctx.n_seqs, ctx.n_decode, ctx.n_logits = n_tokens, n_seqs, n_decode, n_logits
        ctx.token_ids = self._dev("token_ids", n_tokens)
        ctx.positions = self._dev("positions", axes * n_tokens).view(axes, n_tokens)
        ctx.q_start = self._dev("q_start", n_seqs + 1)
        ctx.kv_len = self._dev("kv_len", n_seqs)
        ctx.state_slots = self._dev("state_slots", n_seqs)
        ctx.logit_rows = self._dev("logit_rows", n_logits)
        ctx.groups = [GroupStep(self._dev(f"table{g}", n_seqs * width).view(n_seqs, width),
                                self._dev(f"slots{g}", n_tokens)) for g in range(len(self.cache.pools))]
        ctx.h_q_start = q_start.tolist()
        ctx.h_kv_len = kv_len.tolist()
        ctx.h_state_slots = slots_of.tolist()
        ctx.max_q_len = int(q_lens[n_decode:].max()) if n_decode < n_seqs else 0
        ctx.max_kv_len = int(kv_len.max())
        ctx.kv_capacity = width * page
        ctx.kv_bound = min(ctx.kv_capacity, max(MIN_LENGTH_CLASS, 1 << max(0, ctx.max_kv_len - 1).bit_length()))
        ctx.max_tokens = self.max_tokens
        ctx.cache, ctx.workspace = self.cache, self.workspace
        ctx.token_feed = self.token_feed
        ctx.defer_sums = self._defer_sums

        graphable = (self.use_graphs and n_decode == n_seqs and n_logits == n_seqs
                     and rows == list(range(n_seqs)))
        ctx.capturing = graphable       # fixed launch shapes in warm-up, capture and replay alike
        ctx.staging_index = k
        ctx.staging_segments = segments
        return ctx, ordered, graphable

    def _first_positions(self, group, computed):
        """Per sequence, the first position whose page a windowed group must still hold."""
        window = self.cache.layout.groups[group].spec.window
        if window is None:
            return np.zeros_like(computed)
        return np.maximum(0, computed - window + 1) // self.cache.page_size * self.cache.page_size

    # ---- HIP graphs for decode-only steps ------------------------------------------------
    def _capture(self, ctx):
        """Capture model.forward(ctx) as a chain of graphs.

        Launching a graph costs host time per node before its first kernel starts. With
        `segment_graphs` the step is therefore cut after the first layer run and then every
        GRAPH_SEGMENT_RUNS runs: the first graph is short and starts at once, and every later one
        is launched while its predecessor still runs. A caller that launches a step while the step
        before still runs (the scheduler's lookahead) turns it off: the launch is hidden anyway, and
        every cut costs about 8 us between two graphs.
        """
        lib = library()
        stream = self.stream.cuda_stream
        generation = self.workspace.generation
        handles = []
        n_runs = len(self.model.schedule)

        def end_segment():
            handle = ctypes.c_void_p()
            code = lib.tw_graph_end(stream, ctypes.byref(handle))
            if code == 0:
                handles.append(handle)
            return code

        def segment_end(i):
            if self.segment_graphs and i + 1 < n_runs and (i == 0 or (i + 1) % GRAPH_SEGMENT_RUNS == 0):
                check(end_segment(), "graph capture end")
                check(lib.tw_graph_begin(stream), "graph capture begin")

        check(lib.tw_graph_begin(stream), "graph capture begin")
        ctx.segment_end = segment_end
        self.workspace.touched = touched = set()
        try:
            logits = self.model.forward(ctx)
        except BaseException:
            end_segment()
            for handle in handles:
                lib.tw_graph_destroy(handle)
            raise
        finally:
            ctx.segment_end = None
            self.workspace.touched = None
        check(end_segment(), "graph capture end")
        if self.workspace.generation != generation:
            for handle in handles:
                lib.tw_graph_destroy(handle)
            raise RuntimeError("a scratch buffer was allocated during graph capture")
        return _Graph(handles, logits, generation, {key: self.workspace.versions[key] for key in touched})

    def _run_graphable(self, ctx, key):
        """KEY = (batch size, length class) names the captured graph this step can be replayed from."""
        graph = self._graphs.get(key)
        if graph is not None and graph.generation != self.workspace.generation:
            # some scratch buffer was allocated since: only a capture that holds THAT buffer's address is stale
            if self.workspace.holds(graph.buffers):
                graph.generation = self.workspace.generation
            else:
                self._drop_graph(key)
                graph = None
        if graph is None:
            if key not in self._warm:
                # First time at this batch size and length class: run eagerly so every scratch buffer exists.
                self._warm.add(key)
                return self.model.forward(ctx)
            graph = self._graphs[key] = self._capture(ctx)
            while len(self._graphs) > self.max_graphs:
                self._drop_graph(next(iter(self._graphs)))
        else:
            self._graphs.move_to_end(key)
        lib = library()
        for handle in graph.handles:
            check(lib.tw_graph_launch(handle, self.stream.cuda_stream), "graph launch")
        self.graph_replays += 1
        return graph.logits
