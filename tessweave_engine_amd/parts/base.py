"""Interfaces of the parts a model is assembled from, and what a part sees of a step.

A model is: a token embedding, a list of blocks, a SCHEDULE (the order in which
blocks run: data, not code), a final norm and a head. A block arranges a mixer
(attention here), a feed-forward and norms. Each part gets its sizes and
constants as constructor parameters and never learns which model it is in.

The reference has none of this: its layers are fixed attributes of one class
(flow_engine/model.py:88-102) and its forward is one loop (model.py:176-204).
"""
from __future__ import annotations

from dataclasses import dataclass
import math

import torch


@dataclass(frozen=True)
class LayerRun:
    """One entry of a model's schedule.

    block:        index into the model's blocks (an index may appear more than once)
    cache_slot:   which cache slot the block's mixer uses in this run
    writes_cache: False lets the mixer read a slot that another run wrote in this step
    """
    block: int
    cache_slot: int
    writes_cache: bool = True


class Part:
    """Base of every part: names the checkpoint tensors it owns and takes them over."""

    #: True if `forward` only launches this package's kernels on the current
    #: stream: no host synchronisation, no allocation once buffers exist. Only
    #: models whose parts all say so are replayed from HIP graphs.
    graph_safe = True

    def tensor_specs(self):
        return []

    def bind(self, tensors, dtype, device):
        """Take this part's tensors (already on DEVICE, in their device precision) out of TENSORS."""

    def parts(self):
        """Sub-parts, for walking a model."""
        return []

    def weight_tensors(self):
        """The tensors (torch tensors or kernel-layout weights with `numel()` and `element_size()`) of THIS part,
        not of its sub-parts, that a step reads once in full: matrices, biases, norm weights. What a step only
        gathers rows from (an embedding table) or derives constants from is not among them. The bytes a decode
        step must move, and so its roofline, are counted from this."""
        return []


class Norm(Part):
    #: True if `forward` takes `add`: pending partial sums (float32 [splits, n, hidden]) that the part
    #: before left to be added into x first (see `Mixer.forward`). A model defers such sums only if every
    #: one of its norms says so; a norm that leaves this False is never handed any.
    folds_pending = False

    def forward(self, ctx, x, rows=None):
        """x float32 [n, hidden] -> normalised rows in the compute type.

        rows: int32 indices (on the device) of the rows wanted; None: all of them.
        Norms with `folds_pending` also take add=..., see above.
        """
        raise NotImplementedError


class PositionEncoding(Part):
    """Rotary-style encodings hand per-token (cos, sin) tables to the mixers that use them."""

    rotary_dim = 0
    #: which two elements of a head turn together: "half" pairs element j with j + rotary_dim/2,
    #: "adjacent" pairs element 2j with 2j + 1
    pairing = "half"
    #: position ids a token carries for this encoding: `ctx.positions` is [axes, n_tokens] with as many axes as
    #: the model's encodings ask for at most. Axis 0 counts a request's tokens unless a step entry brings
    #: its own ids; an encoding with one axis reads `ctx.positions[0]`.
    position_axes = 1

    def tables(self, ctx):
        """(cos, sin), float32 [n_tokens, rotary_dim / 2] each, from `ctx.positions`."""
        raise NotImplementedError


class HeadHook(Part):
    """An operation on a mixer's projected heads between bias and rotation (a per-head norm, a scaling).

    `forward(ctx, qkv)` changes qkv [n_tokens, (q_heads + 2 kv_heads) * head_dim] in place, in the compute
    type, on the current stream. The part gets the head counts and sizes it needs as constructor parameters,
    as every part does (head_dim is the size on the device: a multiple of 16, tails of zeros stay zeros).
    """

    def forward(self, ctx, qkv):
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        """A cache.CacheNeed (paged keys/values and/or fixed-size state), or None."""
        return None

    def forward(self, ctx, run, h, x):
        """Add the mixer's output for normalised input H into the residual stream X (float32, in place).

        Returns None, or, only if `ctx.defer_sums` allows it, PENDING partial sums (float32
        [splits, n, hidden]) that are not yet in X: whoever runs next (the following norm) adds them up
        and into X. This saves a kernel per projection when a step has few rows. A part that always
        returns None is a complete part.
        """
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, h, x):
        """Add the feed-forward's output for normalised input H into X (float32, in place);
        returns None or pending partial sums as `Mixer.forward` does."""
        raise NotImplementedError


class Block(Part):
    mixer: Mixer

    def forward(self, ctx, run, x, pending=None):
        """Run the block on X in place. PENDING: partial sums the block before left to be added
        into X; returns what this block leaves pending (or None)."""
        raise NotImplementedError


def fold_pending(x, pending):
    """Add pending partial sums into X with plain tensor operations (for parts written in torch)."""
    if pending is not None:
        x += pending.sum(0)
    return None


class Workspace:
    """Scratch tensors by tag, allocated once and reused by every step."""

    def __init__(self, device):
        self.device = device
        self.buffers = {}
        self.generation = 0          # changes whenever any buffer is (re)allocated
        self.versions = {}           # per buffer: how often it has been (re)allocated
        self.touched = None          # while a set: the buffers asked for (a graph capture notes whose addresses it holds)

    def get(self, tag, shape, dtype, capacity=None):
        """A tensor of SHAPE; the buffer behind it holds CAPACITY rows (default: shape[0])."""
        shape = tuple(int(v) for v in shape)
        numel = math.prod(shape)
        per_row = math.prod(shape[1:]) if shape else 1
        want = max(numel, per_row * max(capacity or 0, shape[0] if shape else 1), 1)
        key = (tag, dtype)
        if self.touched is not None:
            self.touched.add(key)
        buf = self.buffers.get(key)
        if buf is None or buf.numel() < numel:
            buf = torch.empty(want, dtype=dtype, device=self.device)
            self.buffers[key] = buf
            self.versions[key] = self.versions.get(key, 0) + 1
            self.generation += 1
        return buf[:numel].view(shape)

    def holds(self, versions):
        """Are the buffers named in VERSIONS ({key: version}) still the allocations they were then?"""
        return all(self.versions.get(key) == version for key, version in versions.items())

    def bytes(self):
        return sum(b.numel() * b.element_size() for b in self.buffers.values())


class GroupStep:
    """A cache group's metadata for one step."""
    __slots__ = ("block_table", "slot_mapping")

    def __init__(self, block_table, slot_mapping):
        self.block_table = block_table     # int32 [n_seqs, width]; -1 where a block is not held
        self.slot_mapping = slot_mapping   # int32 [n_tokens]; physical token slot of each new token


class StepContext:
    """Everything a part may read during one step.

    The batch is flat: n_tokens rows, grouped by sequence; sequence s owns rows
    q_start[s] .. q_start[s+1]-1, at positions kv_len[s]-q_len .. kv_len[s]-1.
    The first n_decode sequences have exactly one token each.
    """

    def __init__(self):
        self.device = None
        self.dtype = None
        self.n_tokens = 0
        self.n_seqs = 0
        self.n_decode = 0
        self.token_ids = None        # int32 [n_tokens]
        self.positions = None        # int32 [position axes, n_tokens]; axis 0: the token's index in its request
                                     # unless the step entry brought its own ids
        self.q_start = None          # int32 [n_seqs + 1]
        self.kv_len = None           # int32 [n_seqs], this step's tokens included
        self.state_slots = None      # int32 [n_seqs]
        self.logit_rows = None       # int32 [n_logits]
        self.n_logits = 0
        self.groups = []             # GroupStep per cache group
        # host copies, for grid sizes and for parts written in plain torch
        self.h_q_start = []
        self.h_kv_len = []
        self.h_state_slots = []
        self.max_q_len = 0           # over the sequences after the first n_decode
        self.max_kv_len = 0
        self.kv_capacity = 0         # most keys a sequence can ever hold (block-table width * page size)
        self.kv_bound = 0            # while capturing: the step's length class, an upper bound of every kv_len that
                                     # a replay of this capture will see (a power of two, at most kv_capacity)
        self.token_feed = None       # int32 device tensor: a token id -1 - k in token_ids stands for token_feed[k]
        self.defer_sums = True       # may a mixer or feed-forward leave partial sums pending for the next norm?
        self.capturing = False       # launches may depend on kv_bound and capacities, not on this step's lengths
        self.segment_end = None      # while a step is captured: called with the index of each finished layer run
        self.max_tokens = 0          # row capacity of per-token scratch buffers
        self.cache = None            # cache.CacheManager
        self.workspace = None        # Workspace
        self.shared = {}             # per-step values shared by layers (rotary tables, ...)
        self.staging_index = 0       # which host staging buffer holds this step's metadata
        self.staging_segments = None # (offset, words) of the parts of that buffer this step filled

    def scratch(self, tag, shape, dtype=None):
        """Per-token scratch [n, ...]: the buffer is sized once for the largest step."""
        return self.workspace.get(tag, tuple(shape), dtype or self.dtype, capacity=self.max_tokens)
