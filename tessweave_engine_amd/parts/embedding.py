"""Token embedding and the output head (flow_engine/model.py:100,108-112,176,204).

The embedding is a row gather without scaling, into the float32 residual
stream. The head multiplies the normalised rows that were asked for by its
matrix and returns float32 logits; a tied head uses the embedding's matrix and
its own checkpoint key is accepted but never required.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, TensorSpec
from .base import Part


class TokenEmbedding(Part):
    def __init__(self, name, vocab, hidden):
        self.name, self.vocab, self.hidden = name, int(vocab), int(hidden)
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name + ".weight", (self.vocab, self.hidden), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        self.weight = tensors.pop(self.name + ".weight").contiguous()

    def forward(self, ctx):
        x = ctx.scratch("residual", (ctx.n_tokens, self.hidden), torch.float32)
        return ops.embed_gather(ctx.token_ids, self.weight, x, feed=ctx.token_feed)


class OutputHead(Part):
    def __init__(self, name, vocab, hidden, tied_to=None):
        self.name, self.vocab, self.hidden = name, int(vocab), int(hidden)
        self.tied_to = tied_to
        self.weight = None

    def tensor_specs(self):
        if self.tied_to is not None:
            return [TensorSpec(self.name + ".weight", (self.vocab, self.hidden), MATRIX, NORMAL,
                               optional_alias_of=self.tied_to.name + ".weight")]
        return [TensorSpec(self.name + ".weight", (self.vocab, self.hidden), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        # The head's matrix is kept in the matrix kernels' shuffled layout; a tied head makes its own
        # shuffled copy of the embedding (the gather reads rows, the head streams MFMA blocks).
        source = self.tied_to.weight if self.tied_to is not None else tensors.pop(self.name + ".weight").contiguous()
        if torch.device(device).type == "cuda" and ops.can_shuffle(source):
            self.weight = ops.shuffle_weight(source)
        else:
            self.weight = source

    def matrix(self):
        return self.weight

    def weight_tensors(self):
        return [self.weight]          # (the embedding's table is not listed by its part: a step gathers a few rows of it)

    def forward(self, ctx, h):
        # The logits live in a shared scratch buffer: they are valid until the next step.
        logits = ctx.workspace.get("logits", (h.shape[0], self.vocab), torch.float32)
        return ops.linear(h, self.matrix(), logits)
