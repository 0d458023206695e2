"""A decoder model: embedding, blocks run in the order of a schedule, final norm, head."""
from __future__ import annotations

import torch

from ..cache.spec import CacheLayout
from .base import LayerRun, Norm, Part, PositionEncoding
from .blocks import normalise


def walk(part):
    yield part
    for child in part.parts():
        yield from walk(child)


class DecoderModel(Part):
    def __init__(self, config, embedding, blocks, final_norm, head, schedule=None):
        """SCHEDULE defaults to every block once, in order, each with its own cache slot."""
        self.config = config
        self.embedding = embedding
        self.blocks = list(blocks)
        self.final_norm = final_norm
        self.head = head
        self.schedule = list(schedule) if schedule is not None else [LayerRun(i, i) for i in range(len(self.blocks))]
        for run in self.schedule:
            if not 0 <= run.block < len(self.blocks):
                raise ValueError(f"schedule names block {run.block}, the model has {len(self.blocks)}")
        self.dtype = None
        self.device = None
        self._layout = None

    # ---- structure ----------------------------------------------------------
    def parts(self):
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    @property
    def vocab_size(self):
        return self.head.vocab

    @property
    def graph_safe_model(self):
        return all(p.graph_safe for p in walk(self))

    @property
    def defers_sums(self):
        """May mixers and feed-forwards leave split-K sums to the next norm? Only if every norm folds them."""
        return all(p.folds_pending for p in walk(self) if isinstance(p, Norm))

    def tensor_specs(self):
        specs, seen = [], set()
        for part in self.parts():
            for spec in part.tensor_specs():
                if spec.name in seen:
                    raise ValueError(f"two parts claim the tensor {spec.name}")
                seen.add(spec.name)
                specs.append(spec)
        return specs

    def bind(self, tensors, dtype, device):
        tensors = dict(tensors)
        self.dtype, self.device = dtype, torch.device(device)
        for part in self.parts():          # composite parts bind their own sub-parts
            part.bind(tensors, dtype, self.device)
        leftover = [k for k in tensors]
        if leftover:
            raise ValueError(f"tensors no part took: {sorted(leftover)[:12]}")
        return self

    @property
    def position_axes(self):
        """Position ids per token that the step's metadata must carry: the most any of the model's encodings asks for."""
        return max([p.position_axes for p in walk(self) if isinstance(p, PositionEncoding)] + [1])

    def weight_bytes(self):
        """Bytes of every weight a step reads once in full: what the parts name in `weight_tensors()`, each
        allocation counted once (layers may share a part, a tied head has a matrix of its own)."""
        total, seen = 0, set()
        for part in walk(self):
            for t in part.weight_tensors():
                storage = t if isinstance(t, torch.Tensor) else t.data       # (a kernel-layout weight wraps its tensor)
                ident = storage.data_ptr()
                if ident not in seen:
                    seen.add(ident)
                    total += t.numel() * t.element_size()
        return total

    def cache_layout(self):
        """The cache slots the schedule uses and what each holds."""
        if self._layout is None:
            n_slots = max((run.cache_slot for run in self.schedule), default=-1) + 1
            needs = [None] * n_slots
            for run in self.schedule:
                need = self.blocks[run.block].mixer.cache_need()
                if run.writes_cache:
                    if needs[run.cache_slot] is not None and needs[run.cache_slot] != need:
                        raise ValueError(f"cache slot {run.cache_slot} is written with two different needs")
                    needs[run.cache_slot] = need
            for run in self.schedule:
                need = self.blocks[run.block].mixer.cache_need()
                if not run.writes_cache and needs[run.cache_slot] != need:
                    raise ValueError(f"a layer reads cache slot {run.cache_slot}, which holds something else")
            self._layout = CacheLayout(needs)
        return self._layout

    # ---- one step -----------------------------------------------------------------
    def forward(self, ctx):
        """Run the step's tokens; float32 logits [n_logits, vocab] at ctx.logit_rows."""
        x = self.embedding.forward(ctx)
        pending = None              # partial sums a block left for the next norm to add into x
        for i, run in enumerate(self.schedule):
            pending = self.blocks[run.block].forward(ctx, run, x, pending)
            if ctx.segment_end is not None:
                ctx.segment_end(i)
        if ctx.n_logits == 0:
            return torch.empty(0, self.vocab_size, dtype=torch.float32, device=ctx.device)
        h = normalise(self.final_norm, ctx, x, pending, rows=ctx.logit_rows)
        return self.head.forward(ctx, h)
