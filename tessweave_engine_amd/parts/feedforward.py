"""SwiGLU feed-forward: x += down( silu(gate(h)) * up(h) ), no biases (flow_engine/model.py:68-85)."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward
from .linear import Linear


class SwiGLU(FeedForward):
    def __init__(self, prefix, hidden, intermediate, packed=True):
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.gate_up = Linear([prefix + "gate_proj", prefix + "up_proj"], hidden, [intermediate, intermediate],
                              packed=packed)
        self.down = Linear([prefix + "down_proj"], intermediate, [hidden])

    def parts(self):
        return [self.gate_up, self.down]

    def tensor_specs(self):
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, tensors, dtype, device):
        self.gate_up.bind(tensors, dtype, device)
        self.down.bind(tensors, dtype, device)

    def forward(self, ctx, h, x):
        n = h.shape[0]
        gu = ctx.scratch("ffn.gate_up", (n, 2 * self.intermediate))
        self.gate_up.forward(ctx, h, gu)
        if self.down.deferrable(n):
            # few rows: silu(gate) * up is formed while the down projection stages its input,
            # and its split-K sums are left to the next norm
            return self.down.forward_partials(ctx, gu, "down", silu_gate=True)
        # many rows: a separate SiLU-multiply pass (fused into the tiled kernel's tile loads it would
        # be recomputed once per column tile, which costs more than the pass)
        act = ctx.scratch("ffn.act", (n, self.intermediate))
        ops.silu_mul(gu, act)
        self.down.forward(ctx, act, x, residual=x)
        return None
