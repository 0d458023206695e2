"""The cache manager: pages per group, block tables per request, state slots.

For every live request (`Sequence`) it keeps, per group, the list of physical
pages that hold the request's logical blocks (-1 where a block is not held: a
window has passed it, or it is not yet allocated), and one slot index into the
fixed-size state arrays. Position p of a request lives in
`table[p // page_size] * page_size + p % page_size` (flow_engine/cache.py:93-95).

Pages come back when a request closes (flow_engine/engine.py:132-133) and,
for a windowed group, as soon as no later query can see them.
"""
from __future__ import annotations

import math

import numpy as np

from .pages import CapacityError, PagePool, block_keys
from .spec import CacheLayout

_STATE_DTYPES = {"float32": "float32", "bfloat16": "bfloat16", "int32": "int32"}


class Sequence:
    """What the cache holds for one live request."""

    __slots__ = ("id", "state_slot", "tables", "computed", "cached", "promised", "budget", "closed",
                 "block_keys", "key_namespace")

    def __init__(self, seq_id, state_slot, n_groups):
        self.id = seq_id
        self.state_slot = state_slot
        self.tables = [[] for _ in range(n_groups)]   # per group: page id per logical block, -1 = not held
        self.computed = 0                              # tokens whose keys/values (and state) are in the cache
        self.cached = 0                                # tokens taken from the prefix index at admission
        self.promised = [0] * n_groups                 # pages promised to this request and not yet taken
        self.budget = [0] * n_groups                   # pages reserved at admission (0: grows on demand)
        self.closed = False
        self.block_keys = []                           # prefix-index keys of the first full blocks of its tokens, as far
        self.key_namespace = None                      # as they have been hashed (a request's tokens only grow)

    def held(self, group):
        return sum(1 for page in self.tables[group] if page >= 0)


class CacheManager:
    def __init__(self, layout: CacheLayout, page_size, pages, max_requests, dtype="bfloat16",
                 device=None, prefix_cache=True, max_request_tokens=None):
        """PAGES is one count for every group or a list with one count per group.

        MAX_REQUEST_TOKENS bounds one request's length (default: what the
        largest pool could hold); it fixes the width of the block tables.

        DEVICE None keeps only the host-side accounting (no tensors): the
        allocator, tables and slots can be tested without a GPU.
        """
        if page_size <= 0 or max_requests <= 0:
            raise ValueError("page_size and max_requests must be positive")
        self.layout = layout
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        counts = list(pages) if isinstance(pages, (list, tuple)) else [pages] * len(layout.groups)
        if len(counts) != len(layout.groups):
            raise ValueError("one page count per cache group is needed")
        self.prefix_cache = bool(prefix_cache) and layout.shares_prefixes
        self.pools = [PagePool(n, self.page_size, self.prefix_cache) for n in counts]
        if max_request_tokens is None:
            max_request_tokens = max(counts, default=1) * self.page_size
        self.max_request_tokens = int(max_request_tokens)
        self.table_width = max(1, math.ceil(self.max_request_tokens / self.page_size))
        # Block tables as arrays, one row per request slot, kept equal to the
        # requests' page lists; a step gathers its rows from here.
        self.table_rows = [np.full((self.max_requests, self.table_width), -1, dtype=np.int32)
                           for _ in self.pools]
        self.free_state_slots = list(reversed(range(self.max_requests)))
        self.sequences: dict = {}
        self.dtype = dtype
        self.device = device
        self.storage = []       # per group: tensor [slots, 2, pages, kv_heads, page_size, head_dim]
        self.state = {}         # cache slot -> tensor [max_requests, *shape]
        if device is not None:
            self._allocate_storage()

    # ---- device storage -------------------------------------------------
    def _allocate_storage(self):
        import torch
        dtype = getattr(torch, self.dtype) if isinstance(self.dtype, str) else self.dtype
        for group, pool in zip(self.layout.groups, self.pools):
            shape = (len(group.slots), 2, pool.capacity, group.spec.kv_heads, self.page_size,
                     group.spec.head_dim)
            if math.prod(shape) >= 2 ** 40:
                raise ValueError("cache group too large")
            # Uninitialised on purpose (flow_engine/cache.py:22): a page's old
            # contents must never reach a result.
            self.storage.append(torch.empty(shape, dtype=dtype, device=self.device))
        for slot in self.layout.state_slots:
            spec = self.layout.needs[slot].state
            self.state[slot] = torch.zeros((self.max_requests,) + spec.shape,
                                           dtype=getattr(torch, _STATE_DTYPES[spec.dtype]),
                                           device=self.device)

    @property
    def allocated_bytes(self):
        total = sum(t.numel() * t.element_size() for t in self.storage)
        return total + sum(t.numel() * t.element_size() for t in self.state.values())

    def keys_values(self, cache_slot):
        """(keys, values, group index) of CACHE_SLOT; each [pages, kv_heads, page_size, head_dim]."""
        g, i = self.layout.slot_group[cache_slot]
        return self.storage[g][i, 0], self.storage[g][i, 1], g

    # ---- requests ---------------------------------------------------------
    def open(self, seq_id):
        if seq_id in self.sequences:
            raise ValueError(f"request {seq_id!r} is already live")
        if not self.free_state_slots:
            raise CapacityError("no free request slot")
        seq = Sequence(seq_id, self.free_state_slots.pop(), len(self.pools))
        self.sequences[seq_id] = seq
        for slot, tensor in self.state.items():
            tensor[seq.state_slot].zero_()
        return seq

    def pages_needed(self, group, total_tokens, largest_step):
        """Most pages of GROUP a request of TOTAL_TOKENS holds at once."""
        spec = self.layout.groups[group].spec
        full = math.ceil(total_tokens / self.page_size)
        if spec.window is None:
            return full
        # Live positions span at most window - 1 old keys plus one step's tokens;
        # such a span touches at most ceil(span / page) + 1 pages.
        span = spec.window - 1 + max(1, largest_step)
        return min(full, math.ceil(span / self.page_size) + 1)

    def fits(self, total_tokens, largest_step):
        """Could a request of TOTAL_TOKENS ever be admitted (empty cache)?"""
        return all(self.pages_needed(g, total_tokens, largest_step) <= pool.capacity
                   for g, pool in enumerate(self.pools))

    def reserve(self, seq, total_tokens, largest_step):
        """Promise SEQ every page it can need for TOTAL_TOKENS; all groups or none.

        This is the reference's worst-case reservation at admission
        (flow_engine/engine.py:99-105), taken as a promise: the pages are set
        aside now and taken by `ensure` as the request grows.
        """
        done = []
        try:
            for g, pool in enumerate(self.pools):
                want = max(0, self.pages_needed(g, total_tokens, largest_step) - seq.held(g)
                           - seq.promised[g])
                pool.promise(want)
                done.append((g, want))
        except CapacityError:
            for g, want in done:
                self.pools[g].unpromise(want)
            raise
        for g, want in done:
            seq.promised[g] += want
            seq.budget[g] = seq.held(g) + seq.promised[g]

    def acquire_prefix(self, seq, prompt, namespace="local"):
        """Take shared pages for the longest published prefix of PROMPT."""
        if not self.prefix_cache or seq.computed or seq.tables[0]:
            return 0
        pool = self.pools[0]
        shared = pool.acquire_prefix(prompt, namespace, keys=self._keys(seq, prompt, len(prompt) - 1, namespace))
        seq.tables[0] = list(shared)
        self.table_rows[0][seq.state_slot, :len(shared)] = shared
        seq.computed = seq.cached = len(shared) * self.page_size
        return seq.cached

    def admit(self, seq_id, prompt, total_tokens, largest_step, namespace="local"):
        """Open a request, share what the prefix index holds of PROMPT and promise it every further page
        that TOTAL_TOKENS can need. Raises CapacityError, with nothing held and nothing evicted, if a
        request slot or the pages are not to be had now. Prefix hits are counted only for admitted requests
        (flow_engine/engine.py:109)."""
        seq = self.open(seq_id)
        try:
            self.acquire_prefix(seq, prompt, namespace)
            self.reserve(seq, total_tokens, largest_step)
        except CapacityError:
            self.close(seq)
            raise
        if seq.cached:
            self.pools[0].hits += seq.cached
        return seq

    def publish(self, seq, tokens, namespace="local", computed=None):
        """Offer the full blocks of TOKENS that SEQ holds keys and values for (its first COMPUTED tokens,
        by default everything it has computed) to the prefix index."""
        if self.prefix_cache:
            upto = min(seq.computed if computed is None else min(int(computed), seq.computed), len(tokens))
            self.pools[0].publish(tokens, upto, seq.tables[0], namespace, keys=self._keys(seq, tokens, upto, namespace))

    def _keys(self, seq, tokens, upto, namespace):
        """Prefix-index keys of the full blocks of TOKENS[:UPTO]. A request's tokens only grow, so the keys
        hashed for it before stay valid and only the blocks after them are hashed now: a prompt published
        portion by portion is hashed once over, not once per portion."""
        if seq.key_namespace != namespace:
            seq.block_keys, seq.key_namespace = [], namespace
        blocks = max(0, int(upto)) // self.page_size
        if blocks > len(seq.block_keys):
            seq.block_keys = block_keys(tokens[:blocks * self.page_size], self.page_size, namespace, known=seq.block_keys)
        return seq.block_keys[:blocks]

    def first_needed_block(self, group, computed):
        """First logical block of GROUP that a query at position >= COMPUTED can see."""
        window = self.layout.groups[group].spec.window
        if window is None:
            return 0
        return max(0, computed - window + 1) // self.page_size

    def ensure(self, seq, n_tokens):
        """Hold pages for positions [seq.computed, n_tokens) in every group; all or nothing."""
        if seq.closed:
            raise RuntimeError("request is closed")
        if n_tokens > self.max_request_tokens:
            raise ValueError(f"a request may hold at most {self.max_request_tokens} tokens")
        plans = []
        for g, pool in enumerate(self.pools):
            table = seq.tables[g]
            blocks = math.ceil(n_tokens / self.page_size)
            # positions below seq.computed are held already (or a window has passed them)
            first = max(self.first_needed_block(g, seq.computed), seq.computed // self.page_size)
            missing = [b for b in range(first, blocks) if b >= len(table) or table[b] < 0]
            plans.append((g, blocks, missing))
        taken = []
        try:
            for g, blocks, missing in plans:
                from_promise = min(len(missing), seq.promised[g])
                pages = self.pools[g].allocate(len(missing), promised=from_promise)
                taken.append((g, pages, from_promise))
        except CapacityError:
            for g, pages, from_promise in taken:
                self.pools[g].release(pages)
                self.pools[g].promise(from_promise)
            raise
        for (g, blocks, missing), (_, pages, from_promise) in zip(plans, taken):
            table = seq.tables[g]
            table.extend([-1] * (blocks - len(table)))
            for b, page in zip(missing, pages):
                table[b] = page
                self.table_rows[g][seq.state_slot, b] = page
            seq.promised[g] -= from_promise

    def advance(self, seq, computed):
        """Record that the cache now holds COMPUTED tokens; give back pages a window has passed."""
        if computed < seq.computed:
            raise ValueError("a request's computed length cannot shrink")
        seq.computed = computed
        for g, pool in enumerate(self.pools):
            if self.layout.groups[g].spec.window is None:
                continue
            table = seq.tables[g]
            first = min(self.first_needed_block(g, computed), len(table))
            for b in range(first):
                if table[b] >= 0:
                    pool.release([table[b]])
                    table[b] = -1
                    self.table_rows[g][seq.state_slot, b] = -1
                    # A reserved request keeps its budget of simultaneous pages:
                    # the page it gave back is promised to it again.
                    if seq.held(g) + seq.promised[g] < seq.budget[g]:
                        pool.promise(1)
                        seq.promised[g] += 1

    def close(self, seq):
        """Give back everything SEQ holds: pages, promises, its state slot."""
        if seq.closed:
            raise RuntimeError(f"request {seq.id!r} was closed twice")
        for g, pool in enumerate(self.pools):
            pool.release(seq.tables[g])
            pool.unpromise(seq.promised[g])
            seq.tables[g] = []
            seq.promised[g] = 0
            self.table_rows[g][seq.state_slot, :] = -1
        self.free_state_slots.append(seq.state_slot)
        seq.closed = True
        del self.sequences[seq.id]

    def clear_prefixes(self):
        for pool in self.pools:
            pool.clear_prefixes()

    def slot_of(self, seq, group, position):
        """Physical token slot of POSITION (flow_engine/cache.py:93-95)."""
        page = seq.tables[group][position // self.page_size]
        if page < 0:
            raise RuntimeError(f"position {position} of request {seq.id!r} is not held")
        return page * self.page_size + position % self.page_size

    # ---- reports and checks ---------------------------------------------
    def stats(self):
        pool = self.pools[0] if self.pools else None
        out = {"physical_blocks": sum(p.capacity for p in self.pools),
               "free_blocks": sum(len(p.free) for p in self.pools),
               "cached_prefix_blocks": sum(len(p.prefixes) for p in self.pools),
               "prefix_hit_tokens": pool.hits if pool else 0,
               "evictions": sum(p.evictions for p in self.pools),
               "kv_allocated_bytes": self.allocated_bytes,
               "promised_blocks": sum(p.promised for p in self.pools)}
        return out

    def check(self):
        """Raise if any page or slot is lost, held twice or counted wrongly."""
        for g, pool in enumerate(self.pools):
            pool.check([seq.tables[g] for seq in self.sequences.values()])
            promised = sum(seq.promised[g] for seq in self.sequences.values())
            if promised != pool.promised:
                raise AssertionError(f"group {g}: {pool.promised} pages promised, requests hold promises for {promised}")
        for seq in self.sequences.values():
            for g in range(len(self.pools)):
                row = self.table_rows[g][seq.state_slot]
                want = seq.tables[g] + [-1] * (self.table_width - len(seq.tables[g]))
                if row.tolist() != want:
                    raise AssertionError(f"block table row of request {seq.id!r} differs from its page list")
        slots = [seq.state_slot for seq in self.sequences.values()]
        if len(set(slots)) != len(slots):
            raise AssertionError("two requests share a state slot")
        if sorted(slots + self.free_state_slots) != list(range(self.max_requests)):
            raise AssertionError("a state slot is lost or free twice")
