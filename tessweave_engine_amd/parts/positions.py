"""Rotary position encoding, rotate-half pairing (flow_engine/model.py:26-33).

inv_freq[j] = theta^(-2j/rot) is computed on the host in float32 exactly as the
reference writes it; angles, cos and sin are float32 on the device, once per
step for all layers that share this part. `rotary_dim` < head_dim rotates only
the first rotary_dim elements of each head.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import PositionEncoding


class RotaryEmbedding(PositionEncoding):
    def __init__(self, head_dim, theta, rotary_dim=None, pairing="half"):
        if pairing not in ("half", "adjacent"):
            raise ValueError("pairing must be 'half' or 'adjacent'")
        self.pairing = pairing
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim must be even and at most head_dim")
        self.inv_freq = None

    def bind(self, tensors, dtype, device):
        rot = self.rotary_dim
        inv = self.theta ** (-torch.arange(0, rot, 2, dtype=torch.float32) / rot)
        self.inv_freq = inv.to(device)          # a constant the tables are derived from, not a weight

    def tables(self, ctx):
        """(cos, sin), float32 [n_tokens, rotary_dim / 2], computed once per step."""
        key = ("rotary", id(self))
        hit = ctx.shared.get(key)
        if hit is None:
            half = self.rotary_dim // 2
            cos = ctx.scratch(f"rotary.cos.{id(self)}", (ctx.n_tokens, half), torch.float32)
            sin = ctx.scratch(f"rotary.sin.{id(self)}", (ctx.n_tokens, half), torch.float32)
            ops.rope_table(ctx.positions[0], self.inv_freq, cos, sin)
            hit = ctx.shared[key] = (cos, sin)
        return hit


class NoPositionEncoding(PositionEncoding):
    """Mixers given this part rotate nothing."""
    rotary_dim = 0

    def tables(self, ctx):
        return None, None
