"""A linear layer over one or several checkpoint matrices with the same input.

Several matrices are packed by exact row concatenation into one weight, as the
reference packs q,k,v and gate,up (flow_engine/model.py:58-65): 7 matrix
products per layer become 4. `packed=False` keeps them apart (the reference's
`--unfused` ablation, cli.py:73); each then writes its own column range.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, VECTOR, NORMAL, TensorSpec
from .base import Part


def pad_groups(t, dim, unit, to):
    """T with every group of UNIT consecutive entries along DIM followed by TO - UNIT zeros."""
    if to == unit:
        return t
    shape = list(t.shape)
    groups = shape[dim] // unit
    out = t.new_zeros(shape[:dim] + [groups, to] + shape[dim + 1:])
    out.narrow(dim + 1, 0, unit).copy_(t.reshape(shape[:dim] + [groups, unit] + shape[dim + 1:]))
    return out.reshape(shape[:dim] + [groups * to] + shape[dim + 1:])


class Linear(Part):
    def __init__(self, names, in_features, out_features, bias=False, packed=True, glu=False,
                 pad_out=None, pad_in=None):
        """names[i] is the checkpoint prefix of the i-th matrix ("...q_proj"), out_features[i] its rows.

        glu: the two matrices are a gate and an up projection; if they can be packed with their
        rows interleaved (`gated` is then true after bind), `forward_glu` gives silu(gate) * up.
        pad_out = (unit, to): on the device every group of `unit` output rows (a head) is followed by
        `to - unit` rows of zeros (and zero biases), so the layer's output has groups of `to` columns
        whose tail is exactly zero. pad_in = (unit, to): the same for groups of input columns (the
        input then has groups of `to` columns, whose tails meet zeros). The checkpoint's tensors keep
        their own shapes.
        """
        self.names = list(names)
        self.in_features = int(in_features)
        self.out_features = [int(o) for o in out_features]
        self.has_bias = bool(bias)
        self.packed = bool(packed)
        self.glu = bool(glu)
        self.pad_out = tuple(int(v) for v in pad_out) if pad_out and pad_out[0] != pad_out[1] else None
        self.pad_in = tuple(int(v) for v in pad_in) if pad_in and pad_in[0] != pad_in[1] else None
        for pad, sizes in ((self.pad_out, self.out_features), (self.pad_in, [self.in_features])):
            if pad and (pad[1] < pad[0] or any(n % pad[0] for n in sizes)):
                raise ValueError("padded groups must divide the layer's sizes and may only grow")
        self.gated = False
        self.weights = []       # one tensor if packed, else one per name
        self.biases = []
        self._ws_floats = {}

    @property
    def total_out(self):
        return sum(self.out_features)

    def tensor_specs(self):
        specs = []
        for name, rows in zip(self.names, self.out_features):
            specs.append(TensorSpec(name + ".weight", (rows, self.in_features), MATRIX, NORMAL))
            if self.has_bias:
                specs.append(TensorSpec(name + ".bias", (rows,), VECTOR, NORMAL))
        return specs

    def bind(self, tensors, dtype, device):
        weights = [tensors.pop(name + ".weight") for name in self.names]
        biases = [tensors.pop(name + ".bias") for name in self.names] if self.has_bias else []
        if self.pad_out:
            weights = [pad_groups(w, 0, *self.pad_out) for w in weights]
            biases = [pad_groups(b, 0, *self.pad_out) for b in biases]
        if self.pad_in:
            weights = [pad_groups(w, 1, *self.pad_in) for w in weights]
        self.gated = (self.glu and self.packed and len(weights) == 2 and
                      weights[0].shape == weights[1].shape and weights[0].shape[0] % 16 == 0)
        if self.gated:
            weights = [ops.interleave_glu_rows(*weights)]
            biases = [ops.interleave_glu_rows(*biases)] if biases else []
        elif self.packed and len(weights) > 1:
            weights = [torch.cat(weights, 0)]
            biases = [torch.cat(biases, 0)] if biases else []
        # On a GPU the matrices are kept in the kernels' shuffled layout (an exact permutation)
        # whenever their rows are a multiple of 16 bytes; otherwise row-major for the generic kernel.
        on_gpu = torch.device(device).type == "cuda"
        self.weights = [ops.shuffle_weight(w.contiguous()) if on_gpu and ops.can_shuffle(w) else w.contiguous()
                        for w in weights]
        self.biases = [b.contiguous() for b in biases]
        del weights, biases

    def weight_tensors(self):
        return list(self.weights) + list(self.biases)

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in self.weights)

    def row_major(self, i=0):
        """Weight i as a row-major [out, in] tensor (a copy if it is held shuffled; a gated pair keeps its interleaved rows)."""
        w = self.weights[i]
        return w.to_rows() if isinstance(w, ops.ShuffledWeight) else w

    def forward_glu(self, ctx, x, out):
        """out [n, rows of one matrix] = silu(x @ gate.T + b) * (x @ up.T + b), in x's type (needs `gated`)."""
        return ops.linear_glu(x, self.weights[0], out, bias=self.biases[0] if self.biases else None)

    def forward(self, ctx, x, out, residual=None):
        """out[:, columns] = x @ W.T (+ bias) (+ residual); out may be float32 or x's type."""
        if self.gated:
            raise RuntimeError("a gated pair of matrices has interleaved rows; use forward_glu")
        col = 0
        for i, w in enumerate(self.weights):
            rows = w.shape[0]
            target = out if len(self.weights) == 1 else out[:, col:col + rows]
            res = None
            if residual is not None:
                res = residual if len(self.weights) == 1 else residual[:, col:col + rows]
            ws = None
            if x.shape[0] <= 64:
                # Split-K scratch, sized once for the largest skinny batch so it never regrows.
                if i not in self._ws_floats:
                    self._ws_floats[i] = ops.linear_workspace_bytes(w.dtype, 64, rows, w.shape[1]) // 4
                if self._ws_floats[i]:
                    ws = ctx.workspace.get("linear.splitk", (self._ws_floats[i],), torch.float32)
            else:
                # few tiles for the chip (a few hundred rows, or large tiles against a matrix with few
                # columns and a long K): the tiled kernel splits K too
                # (a buffer of its own: growing with a prompt portion, it must not move the one captured decode steps hold)
                floats = ops.linear_workspace_bytes(w.dtype, x.shape[0], rows, w.shape[1]) // 4
                if floats:
                    ws = ctx.workspace.get("linear.splitk.rows", (floats,), torch.float32)
            ops.linear(x, w, target, bias=self.biases[i] if self.biases else None, residual=res, workspace=ws)
            col += rows
        return out

    # ---- leave the split-K sums to the next kernel -------------------------------------------
    def _partial_splits(self, n_rows, lda=None):
        """K ranges of `forward_partials` for N_ROWS rows, LDA elements apart (default: contiguous); 0: none.
        Up to 64 rows the streaming kernels' ranges depend on the matrix and on how many tiles of 16 rows
        there are; above, the tiled kernels choose them per row count and stride."""
        lda = self.weights[0].shape[1] if lda is None else int(lda)
        tile = (n_rows + 15) // 16 * 16 if n_rows <= 64 else n_rows       # up to 64 rows: the same for a tile of 16 rows
        key = ("splits", tile, lda)
        if key not in self._ws_floats:
            self._ws_floats[key] = ops.linear_partial_splits_rows(self.weights[0], tile, lda)
        return self._ws_floats[key]

    def deferrable(self, n_rows):
        """Can `forward_partials` run for N_ROWS rows, and is it worth it? (one packed matrix and a kernel
        that splits K for these rows anyway; a bias is NOT added to the partial sums: the caller's next
        kernel has to, or the caller must not defer)"""
        if len(self.weights) != 1 or n_rows < 1:
            return False
        return self._partial_splits(n_rows) > 0

    def forward_partials(self, ctx, x, tag):
        """float32 [splits, n, out] partial sums of x @ W.T (bias NOT added); see ops.linear_partials."""
        w = self.weights[0]
        n = x.shape[0]
        splits = self._partial_splits(n, x.stride(0) if n > 1 else None)
        if n <= 64:     # sized once for the largest such batch, so that it never regrows under a captured graph
            most = max(self._partial_splits(rows) for rows in (16, 32, 48, 64))
            buf = ctx.workspace.get("linear.partial." + tag, (most, 64, w.shape[0]), torch.float32)
        else:
            buf = ctx.workspace.get("linear.partial.rows." + tag, (splits, n, w.shape[0]), torch.float32)
        partial = buf.view(-1)[:splits * n * w.shape[0]].view(splits, n, w.shape[0])
        return ops.linear_partials(x, w, partial)
