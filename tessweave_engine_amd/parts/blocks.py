"""How a layer's parts are arranged. Pre-norm with two residuals (flow_engine/model.py:179-202):

    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
"""
from __future__ import annotations

from .base import Block


class PreNormBlock(Block):
    def __init__(self, mixer_norm, mixer, ffn_norm, ffn):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype, device):
        for p in self.parts():
            p.bind(tensors, dtype, device)

    def forward(self, ctx, run, x, pending=None):
        h = self.mixer_norm.forward(ctx, x, add=pending)
        pending = self.mixer.forward(ctx, run, h, x)
        h = self.ffn_norm.forward(ctx, x, add=pending)
        return self.ffn.forward(ctx, h, x)
