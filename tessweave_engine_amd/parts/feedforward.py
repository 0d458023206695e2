"""SwiGLU feed-forward: x += down( silu(gate(h)) * up(h) ), no biases (flow_engine/model.py:68-85)."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward
from .linear import Linear


class SwiGLU(FeedForward):
    def __init__(self, prefix, hidden, intermediate, packed=True):
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.gate_up = Linear([prefix + "gate_proj", prefix + "up_proj"], hidden, [intermediate, intermediate],
                              packed=packed, glu=True)
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
        act = ctx.scratch("ffn.act", (n, self.intermediate))
        if self.gate_up.gated:
            # silu(gate) * up is formed in the projection's epilogue; [n, 2 * intermediate] is never stored
            self.gate_up.forward_glu(ctx, h, act)
        else:
            gu = ctx.scratch("ffn.gate_up", (n, 2 * self.intermediate))
            self.gate_up.forward(ctx, h, gu)
            ops.silu_mul(gu, act)
        if ctx.defer_sums and not self.down.biases and self.down.deferrable(n):
            # where the down projection splits K (few rows; many rows against its long K), the sums are left to the next norm
            return self.down.forward_partials(ctx, act, "down")
        self.down.forward(ctx, act, x, residual=x)
        return None
