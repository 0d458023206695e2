"""Grouped-query attention over the paged cache (flow_engine/model.py:36-55,183-201).

q, k, v come from one packed projection (biases optional); q and k are rotated
by the position part; rotated k and raw v go to this run's cache slot; query
head h reads kv head h // (q_heads / kv_heads); scores are scaled by
head_dim^-0.5 unless `scale` says otherwise; the output projection adds into
the residual stream. Sequences with one token use the split-KV decode kernel,
the others the prefill kernel; every dense operation runs once over all rows.
"""
from __future__ import annotations

from ..cache.spec import CacheNeed, PagedKV
from ..kernels import ops
from .base import Mixer
from .linear import Linear

import torch


class GroupedQueryAttention(Mixer):
    def __init__(self, prefix, hidden, q_heads, kv_heads, head_dim, position, qkv_bias=True,
                 o_bias=False, window=None, scale=None, packed=True, head_hook=None, softcap=None):
        """softcap: scaled scores pass through softcap * tanh(score / softcap) before the softmax (the attention
        kernels that take every type and page size then run; the fast bfloat16 ones have no such step).
        head_hook: an optional `HeadHook` that changes the projected q, k, v (bias added) in place before q
        and k are rotated: a per-head norm, a scaling. With a hook the projection is finished by its own
        kernel first (without one, few-row steps leave its split-K sums to the kernel that adds the bias,
        rotates and writes the cache)."""
        if q_heads % kv_heads:
            raise ValueError("q_heads must be a multiple of kv_heads")
        if head_dim % 2 or not 2 <= head_dim <= 256:
            raise ValueError(f"the attention kernels take even head sizes up to 256; head_dim {head_dim} is refused")
        self.prefix = prefix
        self.hidden, self.q_heads, self.kv_heads = int(hidden), int(q_heads), int(kv_heads)
        # The kernels work on heads of a multiple of 16 elements. A head of another size is laid out with a
        # tail of zeros on the device: zero rows in the q/k/v matrices and biases, zero columns in the output
        # matrix. Zero elements add nothing to a score, zero values give zero outputs, which meet zero columns:
        # the result is exactly that of the unpadded head. `head_dim` is the size on the device from here on;
        # the scale and the rotation keep the checkpoint's size.
        self.checkpoint_head_dim = int(head_dim)
        self.head_dim = (int(head_dim) + 15) // 16 * 16
        pad = (self.checkpoint_head_dim, self.head_dim)
        self.position = position
        self.window = window
        self.scale = float(scale) if scale is not None else self.checkpoint_head_dim ** -0.5
        self.softcap = float(softcap) if softcap else 0.0
        self.qkv = Linear([prefix + "q_proj", prefix + "k_proj", prefix + "v_proj"], hidden,
                          [q_heads * head_dim, kv_heads * head_dim, kv_heads * head_dim], bias=qkv_bias, packed=packed,
                          pad_out=pad)
        self.o = Linear([prefix + "o_proj"], q_heads * head_dim, [hidden], bias=o_bias, pad_in=pad)
        self.head_hook = head_hook

    def parts(self):
        return [self.qkv, self.o, self.position] + ([self.head_hook] if self.head_hook is not None else [])

    def tensor_specs(self):
        hook = self.head_hook.tensor_specs() if self.head_hook is not None else []
        return self.qkv.tensor_specs() + self.o.tensor_specs() + hook

    def bind(self, tensors, dtype, device):
        self.qkv.bind(tensors, dtype, device)
        self.o.bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)     # shared by layers; binding again is harmless
        if self.head_hook is not None:
            self.head_hook.bind(tensors, dtype, device)

    def cache_need(self):
        return CacheNeed(paged=PagedKV(self.kv_heads, self.head_dim, self.window))

    def forward(self, ctx, run, h, x):
        n = ctx.n_tokens
        width = (self.q_heads + 2 * self.kv_heads) * self.head_dim
        qkv = ctx.scratch("attn.qkv", (n, width))
        cos, sin = self.position.tables(ctx)
        adjacent = self.position.pairing == "adjacent"
        keys, values, g = ctx.cache.keys_values(run.cache_slot)
        group = ctx.groups[g]
        if n <= 64 and self.head_hook is None and self.qkv.deferrable(n):
            # few rows: the projection leaves split-K sums; bias, rotation and cache write finish them
            partial = self.qkv.forward_partials(ctx, h, "qkv")
            ops.rope_kv_write(qkv, cos, sin, group.slot_mapping, keys, values, self.q_heads, self.kv_heads,
                              self.head_dim, ctx.cache.page_size, write_cache=run.writes_cache,
                              partial=partial, bias=self.qkv.biases[0] if self.qkv.biases else None,
                              adjacent=adjacent)
        else:
            self.qkv.forward(ctx, h, qkv)
            if self.head_hook is not None:
                self.head_hook.forward(ctx, qkv)
            ops.rope_kv_write(qkv, cos, sin, group.slot_mapping, keys, values, self.q_heads, self.kv_heads,
                              self.head_dim, ctx.cache.page_size, write_cache=run.writes_cache, adjacent=adjacent)
        out = ctx.scratch("attn.out", (n, self.q_heads * self.head_dim))
        window = self.window or 0
        if ctx.n_decode:
            # A captured step is replayed for other lengths: its split count follows the step's length
            # class (the kernel itself cuts each sequence's own keys into that many ranges).
            longest = ctx.kv_bound if ctx.capturing else ctx.max_kv_len
            if window:
                longest = min(longest, window)
            splits = ops.attn_decode_splits(ctx.n_decode, self.q_heads, self.kv_heads, longest)
            ws = None
            if splits > 1:
                # sized for the most splits any length class can ask for, so that it never grows under a capture
                most = max(splits, ops.attn_decode_splits(ctx.n_decode, self.q_heads, self.kv_heads,
                                                          min(ctx.kv_capacity, window) if window else ctx.kv_capacity))
                floats = ops.attn_decode_workspace_floats(ctx.n_decode, self.q_heads, self.head_dim, most)
                ws = ctx.workspace.get("attn.split", (floats,), torch.float32)
            ops.attn_decode(qkv, keys, values, group.block_table, ctx.q_start, ctx.kv_len, 0, ctx.n_decode, out,
                            self.q_heads, self.kv_heads, self.head_dim, self.scale, window=window,
                            splits=splits, workspace=ws, softcap=self.softcap)
        if ctx.n_seqs > ctx.n_decode:
            # long key ranges are cut into chunks for separate workgroups when there are few tiles of rows
            longest = min(ctx.max_kv_len, window + ctx.max_q_len) if window else ctx.max_kv_len
            split = ops.attn_prefill_split(ctx.n_seqs - ctx.n_decode, self.q_heads, self.kv_heads, ctx.max_q_len, longest)
            ws = None
            if split[0] > 1:
                ws = ctx.workspace.get("attn.prefill_split", (ops.attn_prefill_workspace_floats(
                    n, self.q_heads, self.head_dim, split[0]),), torch.float32)
            ops.attn_prefill(qkv, keys, values, group.block_table, ctx.q_start, ctx.kv_len, ctx.n_decode,
                             ctx.n_seqs - ctx.n_decode, ctx.max_q_len, out, self.q_heads, self.kv_heads,
                             self.head_dim, self.scale, window=window, split=split, workspace=ws,
                             softcap=self.softcap)
        if ctx.defer_sums and not self.o.biases and self.o.deferrable(n):
            return self.o.forward_partials(ctx, out, "o")          # the next norm adds them into x
        self.o.forward(ctx, out, x, residual=x)
        return None
