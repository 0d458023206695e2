"""RMS norm: y = x * rsqrt(mean(x^2) + eps) * weight (flow_engine/model.py:15-23).

The residual stream it reads is float32; statistics and products are float32
and the result is rounded once to the compute type. The weight is held in
float32 (exact for a bfloat16 checkpoint).
"""
from __future__ import annotations

from ..kernels import ops
from ..weights.spec import VECTOR, ONE_PLUS_NORMAL, TensorSpec
from .base import Norm


class RMSNorm(Norm):
    folds_pending = True

    def __init__(self, name, size, eps):
        self.name = name
        self.size = int(size)
        self.eps = float(eps)
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name + ".weight", (self.size,), VECTOR, ONE_PLUS_NORMAL)]

    def bind(self, tensors, dtype, device):
        self.weight = tensors.pop(self.name + ".weight").contiguous()

    def weight_tensors(self):
        return [self.weight]

    def forward(self, ctx, x, rows=None, add=None):
        tag = "norm.out" if rows is None else "norm.rows"        # a model's last norm (chosen rows) keeps its own buffer
        n_out = rows.numel() if rows is not None else x.shape[0]
        out = ctx.scratch(tag, (n_out, self.size))
        scratch = None
        if add is not None and rows is not None:
            import torch
            scratch = ctx.scratch(tag + ".rows", (n_out, self.size), torch.float32)
        return ops.rmsnorm(x, self.weight, self.eps, out, rows=rows, add=add, row_scratch=scratch)
