"""How a layer's parts are arranged. Pre-norm with two residuals (flow_engine/model.py:179-202):

    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
"""
from __future__ import annotations

from .base import Block, fold_pending


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
        h = normalise(self.mixer_norm, ctx, x, pending)
        pending = self.mixer.forward(ctx, run, h, x)
        h = normalise(self.ffn_norm, ctx, x, pending)
        return self.ffn.forward(ctx, h, x)


def normalise(norm, ctx, x, pending=None, rows=None):
    """NORM of X; PENDING partial sums go to a norm that folds them, and are folded here for one that does not
    (which only happens when parts are driven by hand: a model defers sums only if all its norms fold them)."""
    if pending is not None and not norm.folds_pending:
        pending = fold_pending(x, pending)
    if pending is not None:
        return norm.forward(ctx, x, rows=rows, add=pending)
    return norm.forward(ctx, x, rows=rows)
