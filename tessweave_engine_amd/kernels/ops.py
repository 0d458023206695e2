"""Checked Python entry points of the HIP kernels.

Every function checks on the host that operand shapes, types and strides are
what its kernel and grid assume, then launches on torch's current stream.
Tensors are torch CUDA tensors used as plain device memory; nothing here falls
back to a library routine.
"""
from __future__ import annotations

import torch

from .lib import library, check

F32, BF16 = 0, 1
_DTYPE_ID = {torch.float32: F32, torch.bfloat16: BF16}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need(cond, text):
    if not cond:
        raise ValueError(text)


def _dev(t, dtype=None, name="tensor"):
    _need(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be a CUDA tensor")
    if dtype is not None:
        _need(t.dtype == dtype, f"{name} must be {dtype}, is {t.dtype}")
    return t.data_ptr()


def _rows(t, name):
    """(rows, cols, leading dimension) of a 2-D tensor whose rows are contiguous."""
    _need(t.dim() == 2 and (t.shape[1] == 1 or t.stride(1) == 1), f"{name} must be 2-D with contiguous rows")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    _need(ld >= t.shape[1], f"{name} has overlapping rows")
    return t.shape[0], t.shape[1], ld


def dtype_id(dtype):
    _need(dtype in _DTYPE_ID, f"unsupported dtype {dtype}; float32 and bfloat16 are built")
    return _DTYPE_ID[dtype]


def probe_read(buffer, out, blocks=2048):
    """Launch the plain streaming reader over BUFFER (any contiguous device tensor); returns the bytes it reads.
    A yardstick for benchmarks: time it to get the device's own read ceiling."""
    import ctypes
    _need(buffer.is_contiguous(), "probe_read needs a contiguous buffer")
    n = ctypes.c_long(0)
    check(library().tw_probe_read(_dev(buffer), buffer.numel() * buffer.element_size(), _dev(out, torch.float32, "out"),
                                  int(blocks), ctypes.byref(n), _stream()), "probe_read")
    return int(n.value)


def upload_words(src, dst, segments):
    """dst[o:o + n] = src[o:o + n] for every (o, n) of SEGMENTS (at most 16), by a kernel on the current stream.

    src: a pinned int32 host tensor; dst: an int32 device tensor of the same length. A step's metadata goes to
    the device this way: a copy through the copy engine leaves the compute queue idle around it for tens of
    microseconds, a kernel that reads the pinned memory does not leave the queue."""
    import ctypes
    _need(src.dtype == torch.int32 and dst.dtype == torch.int32 and src.is_contiguous() and dst.is_contiguous(),
          "upload_words moves contiguous int32 buffers")
    _need(src.is_pinned() and dst.is_cuda and src.numel() == dst.numel(), "upload_words: pinned host words to as many device words")
    segments = [(int(o), int(n)) for o, n in segments if n > 0]
    _need(len(segments) <= 16 and all(o >= 0 and o + n <= dst.numel() for o, n in segments), "upload_words: bad segments")
    offsets = (ctypes.c_int * 16)(*[o for o, _ in segments])
    counts = (ctypes.c_int * 16)(*[n for _, n in segments])
    check(library().tw_upload_words(src.data_ptr(), dst.data_ptr(), len(segments), offsets, counts, _stream()), "upload_words")


def embed_gather(ids, table, out, feed=None):
    """out[n, :] = float32(table[ids[n], :]); an id -1 - k stands for feed[k] (int32, on the device)."""
    n = ids.numel()
    vocab, hidden = table.shape
    _need(table.is_contiguous() and out.is_contiguous(), "embedding operands must be contiguous")
    _need(tuple(out.shape) == (n, hidden), "embedding output has the wrong shape")
    check(library().tw_embed_gather(dtype_id(table.dtype), _dev(ids, torch.int32, "ids"), _dev(table),
                                    _dev(out, torch.float32, "out"), n, hidden, vocab,
                                    _dev(feed, torch.int32, "feed") if feed is not None else None,
                                    feed.numel() if feed is not None else 0, _stream()),
          "embed_gather")
    return out


def rmsnorm(x, weight, eps, out, rows=None, add=None, row_scratch=None):
    """out = x * rsqrt(mean(x^2) + eps) * weight per row; x float32, weight float32.

    rows: int32 indices choosing the input row of each output row.
    add: float32 [splits, n, hidden] partial sums first added to x. Without `rows`
    x itself is updated; with `rows` the sums go to row_scratch [n_out, hidden].
    """
    _need(x.dim() == 2 and x.is_contiguous(), "rmsnorm input must be contiguous [n, hidden]")
    n, hidden = x.shape
    n_out = rows.numel() if rows is not None else n
    _need(out.is_contiguous() and tuple(out.shape) == (n_out, hidden), "rmsnorm output has the wrong shape")
    _need(weight.numel() == hidden, "rmsnorm weight has the wrong size")
    add_ptr, splits, stride = None, 0, 0
    scratch_ptr = None
    if add is not None:
        _need(add.dim() == 3 and add.is_contiguous() and tuple(add.shape[1:]) == (n, hidden),
              "rmsnorm partial sums must be [splits, n, hidden]")
        add_ptr, splits, stride = _dev(add, torch.float32, "add"), add.shape[0], n * hidden
        if rows is not None:
            _need(row_scratch is not None and row_scratch.is_contiguous()
                  and tuple(row_scratch.shape) == (n_out, hidden), "rmsnorm with rows and partial sums needs row_scratch [n_out, hidden]")
            scratch_ptr = _dev(row_scratch, torch.float32, "row_scratch")
    check(library().tw_rmsnorm(dtype_id(out.dtype), _dev(x, torch.float32, "x"),
                               _dev(weight, torch.float32, "weight"), _dev(out),
                               _dev(rows, torch.int32, "rows") if rows is not None else None,
                               n_out, hidden, float(eps), add_ptr, splits, stride, scratch_ptr, _stream()), "rmsnorm")
    return out


def rope_table(positions, inv_freq, cos, sin):
    """cos/sin[n, j] of float32(positions[n]) * inv_freq[j]."""
    n, half = positions.numel(), inv_freq.numel()
    _need(cos.is_contiguous() and sin.is_contiguous() and tuple(cos.shape) == (n, half)
          and tuple(sin.shape) == (n, half), "rotary tables must be [n, rot/2]")
    check(library().tw_rope_table(_dev(positions, torch.int32, "positions"),
                                  _dev(inv_freq, torch.float32, "inv_freq"),
                                  _dev(cos, torch.float32, "cos"), _dev(sin, torch.float32, "sin"),
                                  n, half, _stream()), "rope_table")


def rope_kv_write(qkv, cos, sin, slots, keys, values, q_heads, kv_heads, head_dim, page_size,
                  write_cache=True, partial=None, bias=None, adjacent=False):
    """Rotate q (in place) and k of qkv[n] = [q | k | v]; write rotated k and v to the pages.

    Pair j of a head is elements (j, j + rot/2), or with `adjacent` elements (2j, 2j + 1).

    keys [pages, kv_heads, page_size, head_dim]; values hold the same number of
    elements and are written as [pages, kv_heads, head_dim, page_size].
    partial: float32 [splits, n, width] split-K sums of the projection; qkv is then
    first filled with round(sum of the splits + bias).
    """
    n, width, ld = _rows(qkv, "qkv")
    _need(width == (q_heads + 2 * kv_heads) * head_dim, "qkv width does not match the head counts")
    half = cos.shape[1] if cos is not None else 0
    rot = 2 * half
    _need(rot <= head_dim, "rotary dimension exceeds head_dim")
    if rot:
        _need(tuple(cos.shape) == (n, half) and tuple(sin.shape) == (n, half) and cos.is_contiguous()
              and sin.is_contiguous(), "rotary tables must be [n, rot/2]")
    if write_cache:
        _need(keys.dtype == qkv.dtype and values.dtype == qkv.dtype, "cache and qkv types differ")
        _need(keys.is_contiguous() and values.is_contiguous(), "cache tensors must be contiguous")
        _need(tuple(keys.shape[1:]) == (kv_heads, page_size, head_dim), "keys must be [pages, kv_heads, page_size, head_dim]")
        _need(values.numel() == keys.numel(), "keys and values differ in size")
        _need(slots.numel() == n, "one cache slot per token is needed")
    if partial is not None:
        _need(partial.dim() == 3 and partial.is_contiguous() and tuple(partial.shape[1:]) == (n, width),
              "projection partial sums must be [splits, n, width]")
        _need(bias is None or bias.numel() == width, "bias has the wrong size")
    dummy = qkv
    check(library().tw_rope_kv_write(
        dtype_id(qkv.dtype), _dev(qkv), ld,
        _dev(cos, torch.float32, "cos") if rot else _dev(dummy), _dev(sin, torch.float32, "sin") if rot else _dev(dummy),
        _dev(slots, torch.int32, "slots") if write_cache else None,
        _dev(keys) if write_cache else None, _dev(values) if write_cache else None,
        n, q_heads, kv_heads, head_dim, rot, page_size, 1 if write_cache else 0,
        _dev(partial, torch.float32, "partial") if partial is not None else None,
        partial.shape[0] if partial is not None else 0,
        _dev(bias, torch.float32, "bias") if (partial is not None and bias is not None) else None,
        1 if adjacent else 0, _stream()), "rope_kv_write")


def silu_mul(gate_up, out):
    """out[n, i] = silu(gate_up[n, i]) * gate_up[n, inter + i]."""
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gate_up must be contiguous [n, 2*inter]")
    n, inter = gate_up.shape[0], gate_up.shape[1] // 2
    _need(out.is_contiguous() and tuple(out.shape) == (n, inter) and out.dtype == gate_up.dtype,
          "silu_mul output has the wrong shape or type")
    check(library().tw_silu_mul(dtype_id(gate_up.dtype), _dev(gate_up), _dev(out), n, inter, _stream()), "silu_mul")
    return out


class ShuffledWeight:
    """An [n, k] weight in the kernels' own layout: an exact permutation of the matrix, zero padded.

    Blocks of 16 rows x 4 sixteen-byte chunks, stored in the order MFMA fragments are read:
    [ceil(n/16)][k_steps][chunk 0..3][row 0..15][elements of 16 bytes]. One wave-wide load of a
    block is 1 KB of consecutive memory.
    """

    def __init__(self, data, n, k, k_steps, dtype):
        self.data, self.n, self.k, self.k_steps, self.dtype = data, n, k, k_steps, dtype

    @property
    def shape(self):
        return (self.n, self.k)

    def numel(self):
        return self.data.numel()

    def element_size(self):
        return self.data.element_size()

    def to_rows(self):
        """The matrix back in row-major order (for tests)."""
        epf = 16 // self.data.element_size()
        blocks = self.data.view(-1, self.k_steps, 4, 16, epf)
        return blocks.permute(0, 3, 1, 2, 4).reshape(blocks.shape[0] * 16, self.k_steps * 4 * epf)[:self.n, :self.k]


def can_shuffle(weight):
    return weight.dim() == 2 and weight.shape[1] % (16 // weight.element_size()) == 0


def shuffle_weight(weight):
    """The shuffled copy of a row-major [n, k] weight (k must be a multiple of 16 bytes)."""
    _need(can_shuffle(weight), "only weights whose rows are a multiple of 16 bytes can be shuffled")
    n, k = weight.shape
    epf = 16 // weight.element_size()
    k_steps = (k // epf + 3) // 4
    n_pad, k_pad = (n + 15) // 16 * 16, k_steps * 4 * epf
    if (n_pad, k_pad) != (n, k):
        padded = weight.new_zeros((n_pad, k_pad))
        padded[:n, :k] = weight
    else:
        padded = weight
    data = padded.view(n_pad // 16, 16, k_steps, 4, epf).permute(0, 2, 3, 1, 4).contiguous().view(-1)
    return ShuffledWeight(data, n, k, k_steps, weight.dtype)


def _weight_args(weight):
    """(n, k, pointer, ldw, shuffled flag, dtype) of a row-major tensor or a ShuffledWeight."""
    if isinstance(weight, ShuffledWeight):
        return weight.n, weight.k, _dev(weight.data), weight.k_steps, 1, weight.dtype
    n, k, ldw = _rows(weight, "weight")
    return n, k, _dev(weight), ldw, 0, weight.dtype


def linear_workspace_bytes(dtype, max_rows, n, k):
    return int(library().tw_linear_workspace_bytes(dtype_id(dtype), int(max_rows), int(n), int(k)))


def linear_partial_splits(dtype, n, k):
    """K ranges `linear_partials` uses for an [n, k] weight; 0 if the shape is not supported."""
    return int(library().tw_linear_partial_splits(dtype_id(dtype), int(n), int(k)))


def linear_partial_splits_rows(weight, rows, lda=None):
    """K ranges `linear_partials` uses for ROWS rows (LDA elements apart, default: contiguous) against WEIGHT;
    0 where it cannot or would not split (above 64 rows the tiled kernels decide, and split only where whole
    tiles would leave CUs idle; which of them runs depends on the rows' stride too)."""
    n, k, _, _, shuffled, w_dtype = _weight_args(weight)
    return int(library().tw_linear_partial_splits_rows(dtype_id(w_dtype), shuffled, int(rows), n, k,
                                                       int(lda if lda is not None else k)))


def linear_partials(x, weight, partial):
    """partial[s] = x[:, K range s] @ weight[:, K range s].T in float32, for the K ranges
    `linear_partial_splits_rows` names for these rows.

    The caller's next kernel adds the splits up.
    """
    m, kx, lda = _rows(x, "x")
    n, k, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    _need(kx == k, "linear_partials shapes do not agree")
    _need(x.dtype == w_dtype and m >= 1, "linear_partials takes rows of the weight's type")
    splits = linear_partial_splits_rows(weight, m, lda)
    _need(splits > 0, "linear_partials: K must be a multiple of 16 bytes, and above 64 rows the shape must be one the tiled kernels split")
    _need(partial.is_contiguous() and tuple(partial.shape) == (splits, m, n), f"partial must be [{splits}, {m}, {n}]")
    check(library().tw_linear_partials(dtype_id(x.dtype), _dev(x), lda, w_ptr, ldw, shuffled,
                                       _dev(partial, torch.float32, "partial"), partial.numel() * 4, m, n, k,
                                       _stream()), "linear_partials")
    return partial


def interleave_glu_rows(gate, up):
    """[2n, k] with the rows of gate and up [n, k] alternating in blocks of 16 (n a multiple of 16).

    The same order applies to biases ([n] each). This is the row order `linear_glu` expects.
    """
    _need(gate.shape == up.shape and gate.shape[0] % 16 == 0, "gate and up must have equally many rows, a multiple of 16")
    n = gate.shape[0]
    rest = tuple(gate.shape[1:])
    return torch.stack([gate.reshape(n // 16, 16, *rest), up.reshape(n // 16, 16, *rest)], 1).reshape(2 * n, *rest).contiguous()


def linear_glu(x, weight, out, bias=None, force=0):
    """out[m, n/2] = silu(x @ gate.T) * (x @ up.T), weight [n, k] holding gate and up rows
    interleaved by `interleave_glu_rows` (row-major or shuffled); out has x's type."""
    m, k, lda = _rows(x, "x")
    n, k2, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    mo, no, ldc = _rows(out, "out")
    _need(n % 32 == 0, "a gated weight has a multiple of 32 rows")
    _need(k == k2 and mo == m and no == n // 2, f"linear_glu shapes do not agree: x {tuple(x.shape)}, weight {(n, k2)}, out {tuple(out.shape)}")
    _need(x.dtype == w_dtype and out.dtype == x.dtype, "x, weight and out types differ")
    if bias is not None:
        _need(bias.numel() == n, "bias has the wrong size")
    check(library().tw_linear_glu(dtype_id(x.dtype), _dev(x), lda, w_ptr, ldw, shuffled,
                                  _dev(bias, torch.float32, "bias") if bias is not None else None,
                                  _dev(out), ldc, m, n, k, force, _stream()), "linear_glu")
    return out


GEMM_AUTO, GEMM_GENERIC, GEMM_TILED, GEMM_TILED_WIDE, GEMM_SKINNY, GEMM_TILED_256, GEMM_TILED_256X192, GEMM_STREAM_CU = 0, 1, 3, 4, 5, 6, 7, 8


def linear(x, weight, out, bias=None, residual=None, workspace=None, force=GEMM_AUTO):
    """out = x @ weight.T (+ bias) (+ residual).

    x [m, k] and weight [n, k] (a row-major tensor or a ShuffledWeight) share a type (float32 or
    bfloat16); out is float32 (required with a residual; the residual may be `out` itself) or that
    type. bias is float32 [n]; workspace is a float32/byte scratch tensor for split-K.
    """
    m, k, lda = _rows(x, "x")
    n, k2, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    mo, no, ldc = _rows(out, "out")
    _need(k == k2 and mo == m and no == n, f"linear shapes do not agree: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    _need(x.dtype == w_dtype, "x and weight types differ")
    out_f32 = out.dtype == torch.float32
    _need(out_f32 or out.dtype == x.dtype, "out must be float32 or the input type")
    ldr = 0
    if residual is not None:
        _need(out_f32, "a residual needs a float32 output")
        mr, nr, ldr = _rows(residual, "residual")
        _need((mr, nr) == (m, n), "residual shape differs from the output")
    if bias is not None:
        _need(bias.numel() == n and bias.is_contiguous(), "bias has the wrong size")
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(library().tw_linear(dtype_id(x.dtype), 1 if out_f32 else 0, _dev(x), lda, w_ptr, ldw, shuffled,
                              _dev(bias, torch.float32, "bias") if bias is not None else None,
                              _dev(residual, torch.float32, "residual") if residual is not None else None, ldr,
                              _dev(out), ldc, ws_ptr, ws_bytes, m, n, k, int(force), _stream()), "linear")
    return out


def attn_decode_splits(n_seqs, q_heads, kv_heads, max_kv_len):
    return int(library().tw_attn_decode_splits(n_seqs, q_heads, kv_heads, max_kv_len))


def attn_decode_workspace_floats(n_seqs, q_heads, head_dim, splits):
    return int(library().tw_attn_decode_workspace_floats(n_seqs, q_heads, head_dim, splits))


def _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim):
    nq, wq, ldq = _rows(q, "q")
    no, wo, ldo = _rows(out, "out")
    _need(wq >= q_heads * head_dim and wo == q_heads * head_dim and no == nq, "attention q/out shapes do not agree")
    _need(out.dtype == q.dtype == keys.dtype == values.dtype, "attention operand types differ")
    _need(keys.dim() == 4 and keys.is_contiguous() and values.is_contiguous() and values.numel() == keys.numel(),
          "keys must be contiguous [pages, kv_heads, page_size, head_dim] and values the same size")
    _need(keys.shape[1] == kv_heads and keys.shape[3] == head_dim, "cache shape does not match the head sizes")
    _need(head_dim % 16 == 0 and 16 <= head_dim <= 256, "head_dim must be a multiple of 16 between 16 and 256")
    _need(keys.shape[2] % 4 == 0, "page_size must be a multiple of 4")
    _need(q_heads % kv_heads == 0, "q_heads must be a multiple of kv_heads")
    _need(block_table.dim() == 2 and block_table.stride(1) == 1, "block_table must be 2-D")
    _need(q_start.numel() >= kv_len.numel() + 1, "q_start needs one more entry than kv_len")
    return ldq, ldo


def attn_decode(q, keys, values, block_table, q_start, kv_len, seq0, n_seqs, out, q_heads, kv_heads,
                head_dim, scale, window=0, splits=1, workspace=None, generic=False, softcap=0.0):
    """Attention of sequences seq0..seq0+n_seqs-1, each with ONE query token, over their pages.

    generic=True forces the kernel that takes every type and page size (bfloat16 with
    pages of a multiple of 8 keys otherwise runs a faster kernel of its own). softcap > 0 passes the scaled
    scores through softcap * tanh(score / softcap) (that kernel only).
    """
    ldq, ldo = _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim)
    _need(seq0 + n_seqs <= kv_len.numel() and seq0 + n_seqs <= block_table.shape[0], "sequence range exceeds the metadata")
    ws_ptr, ws_floats = None, 0
    if splits > 1:
        _need(workspace is not None and workspace.dtype == torch.float32, "split decode attention needs a float32 workspace")
        ws_ptr, ws_floats = _dev(workspace), workspace.numel()
    check(library().tw_attn_decode(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                   _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                   _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"),
                                   seq0, n_seqs, _dev(out), ldo, ws_ptr, ws_floats, q_heads, kv_heads, head_dim,
                                   keys.shape[2], int(window or 0), float(scale), float(softcap or 0.0), int(splits),
                                   1 if generic else 0, _stream()),
          "attn_decode")
    return out


def attn_prefill_split(n_seqs, q_heads, kv_heads, max_q_len, max_kv_len, tile_rows=0):
    """(max_chunks, kv_chunk, tile_rows): how the fast prefill kernel would cut the keys of a tile into
    chunks that separate workgroups take (max_chunks == 1: not at all) for a launch of this shape, and the
    rows of a workgroup's tile it would use (tile_rows 64 or 128 asks for that size)."""
    import ctypes
    chunk, rows = ctypes.c_int(0), ctypes.c_int(0)
    chunks = int(library().tw_attn_prefill_split(int(n_seqs), q_heads, kv_heads, int(max_q_len), int(max_kv_len),
                                                 int(tile_rows), ctypes.byref(chunk), ctypes.byref(rows)))
    return chunks, int(chunk.value), int(rows.value)


def attn_prefill_workspace_floats(n_tokens, q_heads, head_dim, max_chunks):
    return int(library().tw_attn_prefill_workspace_floats(int(n_tokens), q_heads, head_dim, int(max_chunks)))


def attn_prefill(q, keys, values, block_table, q_start, kv_len, seq0, n_seqs, max_q_len, out, q_heads,
                 kv_heads, head_dim, scale, window=0, generic=False, split=None, workspace=None, softcap=0.0):
    """Attention of sequences seq0..seq0+n_seqs-1 with up to max_q_len query tokens each.

    split = (max_chunks, kv_chunk[, tile_rows]) from attn_prefill_split with a float32 workspace of
    attn_prefill_workspace_floats(rows of q, ...) lets the fast bfloat16 kernel cut long key ranges
    into chunks for separate workgroups (a second kernel merges them in a fixed order).
    """
    ldq, ldo = _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim)
    _need(seq0 + n_seqs <= kv_len.numel() and seq0 + n_seqs <= block_table.shape[0], "sequence range exceeds the metadata")
    max_chunks, kv_chunk, ws_ptr, ws_floats = 1, 0, None, 0
    tile_rows = int(split[2]) if split is not None and len(split) > 2 else 0
    if split is not None and split[0] > 1:
        max_chunks, kv_chunk = int(split[0]), int(split[1])
        _need(workspace is not None and workspace.dtype == torch.float32, "split prefill attention needs a float32 workspace")
        ws_ptr, ws_floats = _dev(workspace), workspace.numel()
    check(library().tw_attn_prefill(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                    _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                    _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"),
                                    seq0, n_seqs, int(max_q_len), _dev(out), ldo, ws_ptr, ws_floats, q.shape[0],
                                    max_chunks, kv_chunk, tile_rows, q_heads, kv_heads, head_dim,
                                    keys.shape[2], int(window or 0), float(scale), float(softcap or 0.0),
                                    1 if generic else 0, _stream()), "attn_prefill")
    return out


def sampling_uniform(seed, counter):
    """The uniform number the sampler draws for (seed, counter); host-side, for tests."""
    return float(library().tw_sampling_uniform(int(seed) & (2 ** 64 - 1), int(counter)))


def sample_workspace_bytes(rows):
    return int(library().tw_sample_workspace_bytes(int(rows)))


def sample_rows(logits, out, temperature=None, seeds=None, counters=None, workspace=None):
    """out[r] = greedy (temperature 0 or None) or sampled token of logits[r].

    workspace: a device tensor of at least sample_workspace_bytes(rows) bytes (allocated here if None).
    """
    rows, vocab, ld = _rows(logits, "logits")
    _need(out.numel() == rows, "one output id per row is needed")
    need = sample_workspace_bytes(rows)
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=logits.device)
    _need(workspace.is_contiguous() and workspace.numel() * workspace.element_size() >= need,
          "the sampling workspace is too small")
    if temperature is not None:
        _need(temperature.numel() == rows and seeds.numel() == rows and counters.numel() == rows,
              "one temperature, seed and counter per row are needed")
        _need(seeds.dtype == torch.int64, "seeds must be int64")
    check(library().tw_sample_rows(_dev(logits, torch.float32, "logits"), ld, rows, vocab,
                                   _dev(temperature, torch.float32, "temperature") if temperature is not None else None,
                                   _dev(seeds) if temperature is not None else None,
                                   _dev(counters, torch.int32, "counters") if temperature is not None else None,
                                   _dev(out, torch.int32, "out"), _dev(workspace),
                                   workspace.numel() * workspace.element_size(), _stream()), "sample_rows")
    return out
