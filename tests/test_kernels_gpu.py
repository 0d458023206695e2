"""Each HIP kernel alone against its plain reference, at sizes other than the engine's."""
import math

import pytest
import torch

import plain_model as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, fp32=(2e-5, 2e-5), bf16=(2e-2, 2e-2)):
    return dict(zip(("atol", "rtol"), fp32 if dtype == torch.float32 else bf16))


@pytest.fixture(scope="module")
def ops(device):
    from tessweave_engine_amd.kernels import ops
    return ops


def rand(shape, dtype, device, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(device)


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_gather(ops, device, dtype):
    table = rand((389, 72), dtype, device)
    ids = torch.tensor([0, 388, 5, 5, 17], dtype=torch.int32, device=device)
    out = torch.empty(5, 72, dtype=torch.float32, device=device)
    ops.embed_gather(ids, table, out)
    torch.testing.assert_close(out, table.float()[ids.long()], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,eps", [(64, 1e-6), (200, 1e-5), (3000, 1e-2), (5120, 1e-5), (8196, 1e-6), (16384, 1e-6),
                                        (16390, 1e-6)])       # one, two and four groups per thread; the generic kernel
def test_rmsnorm(ops, device, dtype, hidden, eps):
    x = rand((7, hidden), torch.float32, device, 3.0)
    w = (1 + rand((hidden,), torch.float32, device, 0.1, seed=1))
    out = torch.empty(7, hidden, dtype=dtype, device=device)
    ops.rmsnorm(x, w, eps, out)
    want = plain.rms_norm(x.cpu().double(), w.cpu().double(), eps).float()
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype, (3e-6, 3e-6), (1e-2, 1e-2)))
    # many rows (another kernel: one wave per row)
    xm = rand((261, hidden), torch.float32, device, 3.0, seed=5)
    outm = torch.full((261, hidden), float("nan"), dtype=dtype, device=device)
    ops.rmsnorm(xm, w, eps, outm)
    wantm = plain.rms_norm(xm.cpu().double(), w.cpu().double(), eps).float()
    torch.testing.assert_close(outm.float().cpu(), wantm, **tol(dtype, (3e-6, 3e-6), (1e-2, 1e-2)))
    # gathered rows
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=device)
    out2 = torch.empty(3, hidden, dtype=dtype, device=device)
    ops.rmsnorm(x, w, eps, out2, rows=rows)
    torch.testing.assert_close(out2, out[rows.long()], atol=0, rtol=0)
    # partial sums folded into x first
    add = rand((3, 7, hidden), torch.float32, device, 1.0, seed=2)
    x2 = x.clone()
    out3 = torch.empty(7, hidden, dtype=dtype, device=device)
    ops.rmsnorm(x2, w, eps, out3, add=add)
    total = x.cpu().double() + add.cpu().double().sum(0)
    torch.testing.assert_close(x2.cpu(), total.float(), atol=1e-5, rtol=1e-6)
    want3 = plain.rms_norm(total, w.cpu().double(), eps).float()
    torch.testing.assert_close(out3.float().cpu(), want3, **tol(dtype, (3e-6, 3e-6), (1e-2, 1e-2)))
    # many rows with partial sums (the wave-per-row kernel's own form of it)
    addm = rand((2, 261, hidden), torch.float32, device, 1.0, seed=6)
    xm2 = xm.clone()
    outm2 = torch.full((261, hidden), float("nan"), dtype=dtype, device=device)
    ops.rmsnorm(xm2, w, eps, outm2, add=addm)
    totalm = xm.cpu().double() + addm.cpu().double().sum(0)
    torch.testing.assert_close(xm2.cpu(), totalm.float(), atol=1e-5, rtol=1e-6)
    torch.testing.assert_close(xm2, (addm[0] + addm[1]) + xm, atol=0, rtol=0)          # in that order, to the bit
    torch.testing.assert_close(outm2.float().cpu(), plain.rms_norm(totalm, w.cpu().double(), eps).float(),
                               **tol(dtype, (3e-6, 3e-6), (1e-2, 1e-2)))
    # gathered rows AND partial sums (a row may be named twice): x itself stays as it was
    rows2 = torch.tensor([6, 0, 6], dtype=torch.int32, device=device)
    x3 = x.clone()
    out4 = torch.empty(3, hidden, dtype=dtype, device=device)
    scratch = torch.empty(3, hidden, dtype=torch.float32, device=device)
    ops.rmsnorm(x3, w, eps, out4, rows=rows2, add=add, row_scratch=scratch)
    torch.testing.assert_close(x3, x, atol=0, rtol=0)
    torch.testing.assert_close(out4, out3[rows2.long()], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,page,theta", [(4, 2, 16, 16, 1e4), (6, 1, 32, 8, 1e6), (5, 5, 48, 4, 5e5),
                                                                 (3, 1, 20, 8, 1e4), (28, 4, 128, 16, 1e6),
                                                                 (4, 2, 32, 12, 1e4), (2, 1, 64, 24, 1e6), (3, 3, 16, 48, 1e4)])
def test_rope_and_cache_write(ops, device, dtype, q_heads, kv_heads, head_dim, page, theta):
    n, pages = 9, 7
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = rand((n, width), dtype, device)
    positions = torch.tensor([0, 1, 2, 500, 501, 37, 1023, 3, 4], dtype=torch.int32, device=device)
    half = head_dim // 2
    inv = (theta ** (-torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim)).to(device)
    cos = torch.empty(n, half, device=device)
    sin = torch.empty(n, half, device=device)
    ops.rope_table(positions, inv, cos, sin)
    keys = torch.full((pages, kv_heads, page, head_dim), float("nan"), dtype=dtype, device=device)
    values = torch.full_like(keys, float("nan"))
    slots = torch.tensor([5 * page + 1, 0, 3 * page + page - 1, -1, 2 * page, 2 * page + 1, 6 * page + 2, 1, 2],
                         dtype=torch.int32, device=device)
    before = qkv.clone()
    ops.rope_kv_write(qkv, cos, sin, slots, keys, values, q_heads, kv_heads, head_dim, page)
    src = before.float().cpu()
    pos = positions.cpu()
    q_want = plain.rope(src[:, :q_heads * head_dim].reshape(n, q_heads, head_dim), pos, theta)
    k_want = plain.rope(src[:, q_heads * head_dim:(q_heads + kv_heads) * head_dim].reshape(n, kv_heads, head_dim), pos, theta)
    v_want = src[:, (q_heads + kv_heads) * head_dim:].reshape(n, kv_heads, head_dim)
    t = tol(dtype, (2e-6, 2e-6), (1e-2, 1e-2))
    torch.testing.assert_close(qkv[:, :q_heads * head_dim].float().cpu().reshape(n, q_heads, head_dim), q_want, **t)
    # v columns of qkv untouched
    torch.testing.assert_close(qkv[:, (q_heads + kv_heads) * head_dim:], before[:, (q_heads + kv_heads) * head_dim:], atol=0, rtol=0)
    kc = keys.float().cpu()
    vc = values.float().cpu().reshape(pages, kv_heads, head_dim, page)      # transposed inside the page
    written = torch.zeros(pages * page, dtype=torch.bool)
    for i, slot in enumerate(slots.tolist()):
        if slot < 0:
            continue
        p, o = divmod(slot, page)
        written[slot] = True
        torch.testing.assert_close(kc[p, :, o, :], k_want[i], **t)
        torch.testing.assert_close(vc[p, :, :, o], v_want[i], atol=0, rtol=0)
    # nothing else was written
    kflat = kc.permute(0, 2, 1, 3).reshape(pages * page, -1)
    assert torch.isnan(kflat[~written]).all()
    vflat = vc.permute(0, 3, 1, 2).reshape(pages * page, -1)
    assert torch.isnan(vflat[~written]).all()
    # rows that are not 16-byte aligned take the kernel that moves one element at a time: identical bits
    wide = torch.zeros(n, width + 1, dtype=dtype, device=device)
    odd = wide[:, :width]
    odd.copy_(before)
    keys1, values1 = torch.full_like(keys, float("nan")), torch.full_like(values, float("nan"))
    ops.rope_kv_write(odd, cos, sin, slots, keys1, values1, q_heads, kv_heads, head_dim, page)
    torch.testing.assert_close(odd, qkv, atol=0, rtol=0)
    torch.testing.assert_close(keys1, keys, atol=0, rtol=0, equal_nan=True)
    torch.testing.assert_close(values1, values, atol=0, rtol=0, equal_nan=True)
    # the same from split-K partial sums plus bias: identical bits
    bias = rand((width,), torch.float32, device, 0.3, seed=9)
    parts = rand((3, n, width), torch.float32, device, 1.0, seed=10)
    summed = ((parts[0] + parts[1] + parts[2]) + bias).to(dtype)
    keys2, values2 = torch.zeros_like(keys), torch.zeros_like(values)
    ops.rope_kv_write(summed.clone(), cos, sin, slots, keys2, values2, q_heads, kv_heads, head_dim, page)
    qkv3 = torch.full((n, width), float("nan"), dtype=dtype, device=device)
    keys3, values3 = torch.zeros_like(keys), torch.zeros_like(values)
    ops.rope_kv_write(qkv3, cos, sin, slots, keys3, values3, q_heads, kv_heads, head_dim, page, partial=parts, bias=bias)
    torch.testing.assert_close(keys3, keys2, atol=0, rtol=0)
    torch.testing.assert_close(values3, values2, atol=0, rtol=0)
    ref = summed.clone()
    ops.rope_kv_write(ref, cos, sin, slots, torch.zeros_like(keys), torch.zeros_like(values), q_heads, kv_heads, head_dim, page)
    torch.testing.assert_close(qkv3[:, :q_heads * head_dim], ref[:, :q_heads * head_dim], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kv_heads,head_dim,page", [(2, 32, 16), (4, 128, 16), (1, 64, 8), (3, 48, 32), (2, 32, 4),
                                                    (2, 32, 12), (1, 64, 24), (2, 16, 48), (1, 128, 20)])
def test_cache_write_of_tokens_with_consecutive_slots(ops, device, dtype, kv_heads, head_dim, page):
    """A prompt portion holds consecutive slots: aligned groups of them write the transposed value pages
    together. Runs that start and end anywhere, a gap, a row that writes nothing and rows in other pages
    must leave exactly what the element-wise kernel leaves."""
    q_heads = 2 * kv_heads
    width = (q_heads + 2 * kv_heads) * head_dim
    pages = 40
    runs = [(3, 45), (72, 16), (97, 3)]                              # (first slot, tokens)
    slots = [s for first, count in runs for s in range(first, first + count)]
    slots[20] = -1                                                   # a row in the middle of a run writes nothing
    slots += [130, 120, 122]                                         # single tokens elsewhere
    n = len(slots)
    slots_t = torch.tensor(slots, dtype=torch.int32, device=device)
    qkv = rand((n, width), dtype, device)
    half = head_dim // 2
    positions = torch.arange(n, dtype=torch.int32, device=device)
    inv = (1e4 ** (-torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim)).to(device)
    cos, sin = torch.empty(n, half, device=device), torch.empty(n, half, device=device)
    ops.rope_table(positions, inv, cos, sin)
    results = []
    for pad in (0, 1):                                               # rows of odd length take the element-wise kernel
        buf = torch.zeros(n, width + pad, dtype=dtype, device=device)
        rows = buf[:, :width]
        rows.copy_(qkv)
        keys = torch.full((pages, kv_heads, page, head_dim), float("nan"), dtype=dtype, device=device)
        values = torch.full_like(keys, float("nan"))
        ops.rope_kv_write(rows, cos, sin, slots_t, keys, values, q_heads, kv_heads, head_dim, page)
        results.append((rows.clone(), keys, values))
    for a, b in zip(*results):
        torch.testing.assert_close(a, b, atol=0, rtol=0, equal_nan=True)
    values = results[0][2].float().cpu().reshape(pages, kv_heads, head_dim, page)
    v_src = qkv[:, (q_heads + kv_heads) * head_dim:].float().cpu().reshape(n, kv_heads, head_dim)
    written = torch.zeros(pages * page, dtype=torch.bool)
    for i, slot in enumerate(slots):
        if slot >= 0:
            written[slot] = True
            torch.testing.assert_close(values[slot // page, :, :, slot % page], v_src[i], atol=0, rtol=0)
    assert torch.isnan(values.permute(0, 3, 1, 2).reshape(pages * page, -1)[~written]).all()


@pytest.mark.parametrize("theta", [1e4, 1e6])
def test_rope_tables_at_far_positions(ops, device, theta):
    """cos and sin of float32(position) * inv_freq at positions up to 131,071: the angle is formed in float32 as
    the reference forms it (flow_engine/model.py:28-29), and the fast pairs turn tens of thousands of times."""
    positions = torch.tensor([0, 1, 4095, 4096, 31999, 32767, 32768, 100003, 131071], dtype=torch.int32)
    inv = theta ** (-torch.arange(0, 128, 2, dtype=torch.float32) / 128)
    cos = torch.empty(len(positions), 64, device=device)
    sin = torch.empty_like(cos)
    ops.rope_table(positions.to(device), inv.to(device), cos, sin)
    angle = positions.float()[:, None] * inv[None, :]                       # float32, as the kernel
    torch.testing.assert_close(cos.cpu(), angle.double().cos().float(), atol=3e-7, rtol=0)
    torch.testing.assert_close(sin.cpu(), angle.double().sin().float(), atol=3e-7, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,rot", [(16, 16), (32, 12), (48, 48)])
def test_rope_with_adjacent_pairs(ops, device, dtype, head_dim, rot):
    """Pairs (2j, 2j + 1) instead of (j, j + rot/2): the same rotation applied to the de-interleaved head."""
    n, q_heads, kv_heads, page, pages, theta = 6, 3, 1, 4, 5, 1e4
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = rand((n, width), dtype, device)
    positions = torch.tensor([0, 1, 7, 300, 301, 2], dtype=torch.int32, device=device)
    inv = (theta ** (-torch.arange(0, rot, 2, dtype=torch.float32) / rot)).to(device)
    cos, sin = torch.empty(n, rot // 2, device=device), torch.empty(n, rot // 2, device=device)
    ops.rope_table(positions, inv, cos, sin)
    slots = torch.tensor([4, 5, 0, 19, 9, 13], dtype=torch.int32, device=device)
    src = qkv.float().cpu()

    def want(block, heads):
        x = block.reshape(n, heads, head_dim)
        head = x[..., :rot]
        halves = torch.cat((head[..., 0::2], head[..., 1::2]), -1)              # (2j, 2j + 1) -> (j, j + rot/2)
        turned = plain.rope(halves, positions.cpu(), theta)
        back = torch.empty_like(head)
        back[..., 0::2], back[..., 1::2] = turned[..., :rot // 2], turned[..., rot // 2:]
        return torch.cat((back, x[..., rot:]), -1)
    q_want = want(src[:, :q_heads * head_dim], q_heads)
    k_want = want(src[:, q_heads * head_dim:(q_heads + kv_heads) * head_dim], kv_heads)
    t = tol(dtype, (2e-6, 2e-6), (1e-2, 1e-2))
    bias = rand((width,), torch.float32, device, 0.3, seed=9)
    for from_partials in (False, True):
        keys = torch.zeros((pages, kv_heads, page, head_dim), dtype=dtype, device=device)
        values = torch.zeros_like(keys)
        if from_partials:                       # the same from split-K sums (no bias here: zeros)
            parts = torch.stack([qkv.float() * 0.25, qkv.float() * 0.75])
            got = torch.full((n, width), float("nan"), dtype=dtype, device=device)
            ops.rope_kv_write(got, cos, sin, slots, keys, values, q_heads, kv_heads, head_dim, page, partial=parts,
                              bias=torch.zeros_like(bias), adjacent=True)
        else:
            got = qkv.clone()
            ops.rope_kv_write(got, cos, sin, slots, keys, values, q_heads, kv_heads, head_dim, page, adjacent=True)
        torch.testing.assert_close(got[:, :q_heads * head_dim].float().cpu().reshape(n, q_heads, head_dim), q_want, **t)
        kc = keys.float().cpu()
        for i, slot in enumerate(slots.tolist()):
            torch.testing.assert_close(kc[slot // page, :, slot % page, :], k_want[i], **t)
    half_form = qkv.clone()
    ops.rope_kv_write(half_form, cos, sin, slots, torch.zeros_like(keys), torch.zeros_like(values), q_heads, kv_heads,
                      head_dim, page)
    assert not torch.allclose(half_form[:, :q_heads * head_dim].float().cpu().reshape(n, q_heads, head_dim), q_want, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, device, dtype):
    gu = rand((5, 2 * 70), dtype, device, 2.0)
    out = torch.empty(5, 70, dtype=dtype, device=device)
    ops.silu_mul(gu, out)
    g, u = gu.float().cpu()[:, :70], gu.float().cpu()[:, 70:]
    torch.testing.assert_close(out.float().cpu(), torch.nn.functional.silu(g) * u, **tol(dtype, (1e-6, 1e-6), (1e-2, 1e-2)))


# ---------------------------------------------------------------------------------------
LINEAR_SHAPES = [  # m, n, k
    (1, 16, 64), (3, 389, 320), (8, 1000, 1032), (16, 48, 4096), (17, 130, 192), (33, 64, 8200),
    (64, 256, 512), (65, 200, 136), (130, 389, 64), (300, 520, 776),
    (130, 96, 4096), (257, 260, 2056),      # few tiles, long K: the tiled kernel splits K as well
    (300, 520, 800), (513, 300, 4128),      # K a multiple of 32: the larger tiles copy straight into LDS
    (8, 18950, 64), (16, 18944, 32),        # few rows, one K range, many columns: workgroups of two waves
    (40, 9000, 256), (64, 45000, 96), (20, 2000, 1536), (48, 520, 9472),   # one workgroup per CU: rounds, K ranges, an idle wave
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", LINEAR_SHAPES)
def test_linear_all_paths(ops, device, dtype, m, n, k):
    x = rand((m, k), dtype, device, 1.0, seed=1)
    w = rand((n, k), dtype, device, 0.05, seed=2)
    bias = rand((n,), torch.float32, device, 0.5, seed=3)
    res = rand((m, n), torch.float32, device, 1.0, seed=4)
    want = x.double().cpu() @ w.double().cpu().T
    ws_bytes = max(ops.linear_workspace_bytes(dtype, m, n, k), 16 * 64 * n * 4)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=device)
    forces = [ops.GEMM_AUTO, ops.GEMM_GENERIC, ops.GEMM_TILED, ops.GEMM_TILED_WIDE]
    if m <= 64:
        forces += [ops.GEMM_SKINNY]
    scale = math.sqrt(k) * 0.05
    t = dict(atol=2e-5 * scale, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2 * scale, rtol=2e-2)
    shuffled = ops.shuffle_weight(w)
    torch.testing.assert_close(shuffled.to_rows(), w, atol=0, rtol=0)          # an exact permutation
    big = (ops.GEMM_TILED_256, ops.GEMM_TILED_256X192) if dtype == torch.bfloat16 else ()   # bfloat16, shuffled weights
    if not big:                                                        # ... and refused otherwise
        with pytest.raises(Exception, match="refused its arguments"):
            ops.linear(x, shuffled, torch.empty((m, n), dtype=dtype, device=device), force=ops.GEMM_TILED_256)
    for force in forces + [("shuffled", f) for f in (ops.GEMM_AUTO, ops.GEMM_GENERIC, ops.GEMM_TILED, ops.GEMM_TILED_WIDE)
                           + big + ((ops.GEMM_SKINNY, ops.GEMM_STREAM_CU) if m <= 64 else ())]:
        wt = w
        if isinstance(force, tuple):
            wt, force = shuffled, force[1]
        w_rows, w = w, wt
        # plain output in the input type
        out = torch.full((m, n), float("nan"), dtype=dtype, device=device)
        ops.linear(x, w, out, workspace=ws, force=force)
        torch.testing.assert_close(out.double().cpu(), want, **t)
        # bias + residual into a float32 output that is also the residual
        acc = res.clone()
        ops.linear(x, w, acc, bias=bias, residual=acc, workspace=ws, force=force)
        torch.testing.assert_close(acc.double().cpu(), want + bias.double().cpu() + res.double().cpu(),
                                   atol=t["atol"] if dtype == torch.float32 else 2e-5 * scale + 1e-5, rtol=1e-5)
        # without workspace (no split-K)
        out2 = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
        ops.linear(x, w, out2, bias=bias, force=force)
        torch.testing.assert_close(out2.double().cpu(), want + bias.double().cpu(),
                                   atol=t["atol"] if dtype == torch.float32 else 2e-5 * scale + 1e-5, rtol=1e-5)
        w = w_rows


@pytest.mark.parametrize("m,n,k", [(1024, 3584, 16384), (1100, 3000, 12288), (2048, 3584, 8192)])
def test_linear_large_tiles_over_k_ranges(ops, device, m, n, k):
    """Many rows, few columns, long K (a down projection): the chosen plan may be 256x256 tiles whose K is
    dealt to two to four workgroups, finished by the reduction kernel; with and without workspace."""
    dtype = torch.bfloat16
    x = rand((m, k), dtype, device, 1.0, seed=1)
    w = rand((n, k), dtype, device, 0.05, seed=2)
    bias = rand((n,), torch.float32, device, 0.5, seed=3)
    res = rand((m, n), torch.float32, device, 1.0, seed=4)
    want = (x.double() @ w.double().T).cpu()
    shuffled = ops.shuffle_weight(w)
    ws_bytes = ops.linear_workspace_bytes(dtype, m, n, k)
    assert ws_bytes >= (2 * m * n * 4 if k >= 12288 else 0)      # long K: at least two K ranges are planned
    ws = torch.empty(max(ws_bytes, 16) // 4, dtype=torch.float32, device=device)
    scale = math.sqrt(k) * 0.05
    for workspace in (ws, None):
        out = torch.full((m, n), float("nan"), dtype=dtype, device=device)
        ops.linear(x, shuffled, out, workspace=workspace)
        torch.testing.assert_close(out.double().cpu(), want, atol=2e-2 * scale, rtol=2e-2)
        acc = res.clone()
        ops.linear(x, shuffled, acc, bias=bias, residual=acc, workspace=workspace)
        torch.testing.assert_close(acc.double().cpu(), want + bias.double().cpu() + res.double().cpu(),
                                   atol=2e-5 * scale + 1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 389, 2048), (17, 130, 4096), (64, 96, 9472), (33, 4608, 3584),
                                   (64, 3584, 2368), (48, 1000, 520)])
def test_linear_partials(ops, device, dtype, m, n, k):
    """Sums of K ranges left for the next kernel: row-major weights through the kernel with four column tiles a
    workgroup, shuffled ones through the same (up to 16 rows: identical bits) or, above 16 rows, through the
    kernel with one workgroup per CU, which names its own number of ranges."""
    x = rand((m, k), dtype, device, 1.0, seed=1)
    w = rand((n, k), dtype, device, 0.05, seed=2)
    want = x.double().cpu() @ w.double().cpu().T
    scale = math.sqrt(k) * 0.05
    sums = []
    for weight in (w, ops.shuffle_weight(w)):
        splits = ops.linear_partial_splits_rows(weight, m)
        assert splits >= 1
        part = torch.full((splits, m, n), float("nan"), device=device)
        ops.linear_partials(x, weight, part)
        torch.testing.assert_close(part.double().sum(0).cpu(), want, atol=3e-5 * scale, rtol=1e-5)
        if k >= 2048:
            assert part.abs().amax(dim=(1, 2)).min() > 0         # every range did its share
        with pytest.raises(ValueError, match="partial must be"):
            ops.linear_partials(x, weight, torch.empty(splits + 1, m, n, device=device))
        sums.append(part.sum(0).clone())
    if m <= 16:
        assert ops.linear_partial_splits_rows(w, m) == ops.linear_partial_splits(dtype, n, k)
        torch.testing.assert_close(sums[0], sums[1], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(300, 256, 4096), (1024, 512, 8192), (2048, 896, 9472), (520, 130, 2056),
                                   (2048, 4096, 512)])
def test_linear_partials_of_many_rows(ops, device, dtype, m, n, k):
    """Above 64 rows the tiled kernels leave the sums of their K ranges; where they would not split K
    the call is refused (the product with its epilogue is then the better one)."""
    x = rand((m, k), dtype, device, 1.0, seed=1)
    w = rand((n, k), dtype, device, 0.05, seed=2)
    want = (x.double() @ w.double().T).cpu()
    scale = math.sqrt(k) * 0.05
    seen = 0
    wide = torch.zeros(m, k + 48, dtype=dtype, device=device)      # the same rows, 48 elements further apart
    wide[:, :k] = x
    for weight, rows in ((w, x), (ops.shuffle_weight(w), x), (ops.shuffle_weight(w), wide[:, :k])):
        splits = ops.linear_partial_splits_rows(weight, m, rows.stride(0))
        if splits == 0:
            with pytest.raises(ValueError, match="linear_partials"):
                ops.linear_partials(rows, weight, torch.empty(1, m, n, device=device))
            continue
        assert splits >= 2
        seen += 1
        part = torch.full((splits, m, n), float("nan"), device=device)
        ops.linear_partials(rows, weight, part)
        torch.testing.assert_close(part.double().sum(0).cpu(), want, atol=3e-5 * scale, rtol=1e-5)
        assert part.abs().amax(dim=(1, 2)).min() > 0             # every range did its share
        with pytest.raises(ValueError, match="partial must be"):
            ops.linear_partials(rows, weight, torch.empty(splits + 1, m, n, device=device))
    assert seen or (m, n, k) == (2048, 4096, 512)                # (many tiles, short K: nothing to split)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,inter,k", [(1, 16, 64), (8, 208, 320), (17, 48, 1032), (64, 1040, 256), (65, 80, 64),
                                       (200, 400, 320), (130, 16, 101), (520, 272, 200), (520, 272, 320),
                                       (8, 9472, 64), (3, 9488, 96),      # so many columns that few rows run in workgroups of two waves
                                       (33, 2400, 128), (64, 18944, 96), (50, 176, 512)])   # one workgroup per CU: pairs in rounds
def test_linear_glu(ops, device, dtype, m, inter, k):
    """silu(x gate^T + b) * (x up^T + b) from interleaved rows, every kernel and both layouts."""
    x = rand((m, k), dtype, device, 1.0, seed=1)
    gate, up = rand((inter, k), dtype, device, 0.08, seed=2), rand((inter, k), dtype, device, 0.08, seed=3)
    bg, bu = rand((inter,), torch.float32, device, 0.5, seed=4), rand((inter,), torch.float32, device, 0.5, seed=5)
    w = ops.interleave_glu_rows(gate, up)
    bias = ops.interleave_glu_rows(bg, bu)
    assert torch.equal(w[:16], gate[:16]) and torch.equal(w[16:32], up[:16])
    xd = x.double().cpu()
    scale = math.sqrt(k) * 0.08
    t = dict(atol=3e-5 * scale, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2 * scale, rtol=2e-2)
    aligned = k % (16 // x.element_size()) == 0
    forces = [ops.GEMM_AUTO, ops.GEMM_GENERIC] + ([ops.GEMM_TILED, ops.GEMM_TILED_WIDE] if aligned else [])
    if m <= 64 and aligned:
        forces.append(ops.GEMM_SKINNY)
    layouts = [w] + ([ops.shuffle_weight(w)] if aligned else [])
    for b in (None, bias):
        g = xd @ gate.double().cpu().T + (bg.double().cpu() if b is not None else 0)
        u = xd @ up.double().cpu().T + (bu.double().cpu() if b is not None else 0)
        want = torch.nn.functional.silu(g) * u
        for weight in layouts:
            big = [ops.GEMM_TILED_256, ops.GEMM_TILED_256X192] if (dtype == torch.bfloat16 and weight is not w) else []
            if weight is not w and m <= 64:
                big = big + [ops.GEMM_STREAM_CU]
            for force in forces + big:
                out = torch.full((m, inter), float("nan"), dtype=dtype, device=device)
                ops.linear_glu(x, weight, out, bias=b, force=force)
                torch.testing.assert_close(out.double().cpu(), want, **t)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_odd_k_uses_generic(ops, device, dtype):
    m, n, k = 5, 37, 101
    x, w = rand((m, k), dtype, device, seed=1), rand((n, k), dtype, device, 0.1, seed=2)
    out = torch.empty(m, n, dtype=torch.float32, device=device)
    ops.linear(x, w, out)
    torch.testing.assert_close(out.double().cpu(), x.double().cpu() @ w.double().cpu().T, atol=1e-4, rtol=1e-5)


def test_linear_strided_input_view(ops, device):
    # the activation may be a column slice of a wider buffer
    buf = rand((20, 256), torch.bfloat16, device, seed=5)
    x = buf[:, 64:192]
    w = rand((48, 128), torch.bfloat16, device, 0.1, seed=6)
    out = torch.empty(20, 48, dtype=torch.float32, device=device)
    ops.linear(x, w, out)
    torch.testing.assert_close(out.double().cpu(), x.double().cpu() @ w.double().cpu().T, atol=1e-4, rtol=1e-5)


# ---------------------------------------------------------------------------------------
def build_paged(k, v, lengths, page, pages_total, device, dtype, seed=0, poison=True):
    """Scatter per-sequence k, v [len, Hk, D] into shuffled pages; returns keys, values, table."""
    hk, d = k[0].shape[1], k[0].shape[2]
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(pages_total, generator=g).tolist()
    fill = float("nan") if poison else 0.0
    keys = torch.full((pages_total, hk, page, d), fill, dtype=torch.float32)
    values = torch.full((pages_total, hk, d, page), fill, dtype=torch.float32)
    width = max(math.ceil(n / page) for n in lengths) + 1
    table = torch.full((len(lengths), width), -1, dtype=torch.int32)
    used = 0
    for s, n in enumerate(lengths):
        for b in range(math.ceil(n / page)):
            pg = perm[used]
            used += 1
            table[s, b] = pg
            lo, hi = b * page, min(n, (b + 1) * page)
            keys[pg, :, :hi - lo, :] = k[s][lo:hi].permute(1, 0, 2)
            values[pg, :, :, :hi - lo] = v[s][lo:hi].permute(1, 2, 0)
    return keys.to(dtype).to(device), values.to(dtype).to(device).reshape(pages_total, hk, page, d), table.to(device)


ATTN_TOL = {torch.float32: dict(atol=3e-5, rtol=3e-5), torch.bfloat16: dict(atol=.025, rtol=.025)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim", [16, 32, 48, 64, 80, 128, 256])
@pytest.mark.parametrize("heads,kv_heads", [(8, 8), (8, 2), (8, 1), (28, 4), (40, 2)])
def test_attn_decode_matrix(ops, device, dtype, head_dim, heads, kv_heads):
    """The reference's kernel gate (tools/validate_cuda.py:25-52): ragged lengths, shuffled pages."""
    if head_dim in (48, 80) and (heads, kv_heads) not in ((8, 2), (28, 4)):
        pytest.skip("odd head sizes are run on two head layouts")
    lengths, page = [1, 17, 65, 257], 16
    torch.manual_seed(20261008)
    k = [torch.randn(n, kv_heads, head_dim).to(dtype).float() for n in lengths]
    v = [torch.randn(n, kv_heads, head_dim).to(dtype).float() for n in lengths]
    q = torch.randn(len(lengths), heads, head_dim).to(dtype)
    keys, values, table = build_paged(k, v, lengths, page, 80, device, dtype)
    want = torch.stack([plain.attention(q[i:i + 1].float(), k[i], v[i], torch.tensor([lengths[i] - 1]))[0]
                        for i in range(len(lengths))])
    qd = q.reshape(len(lengths), heads * head_dim).to(device)
    q_start = torch.arange(len(lengths) + 1, dtype=torch.int32, device=device)
    kv_len = torch.tensor(lengths, dtype=torch.int32, device=device)
    for splits, generic in ((1, False), (2, False), (5, False), (1, True), (3, True)):
        out = torch.full((len(lengths), heads * head_dim), float("nan"), dtype=dtype, device=device)
        ws = torch.empty(max(1, ops.attn_decode_workspace_floats(len(lengths), heads, head_dim, splits)), device=device)
        ops.attn_decode(qd, keys, values, table, q_start, kv_len, 0, len(lengths), out, heads, kv_heads,
                        head_dim, head_dim ** -0.5, splits=splits, workspace=ws, generic=generic)
        torch.testing.assert_close(out.float().cpu().reshape(len(lengths), heads, head_dim), want, **ATTN_TOL[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_reference_vector_tables(ops, device, dtype):
    """tests/test_engine.py:288-307 of the reference: tables [[3,1,6],[4,7]], lengths [37,19], 8 q heads on 2."""
    torch.manual_seed(5)
    dim, page = 64, 16
    q = torch.randn(2, 8, dim).to(dtype)
    kpool = torch.randn(8, page, 2, dim).to(dtype)       # the reference's [pages, page, kv, d] layout
    vpool = torch.randn(8, page, 2, dim).to(dtype)
    tables, lengths = [[3, 1, 6], [4, 7]], [37, 19]
    want = []
    for i in range(2):
        kk = kpool[tables[i]].flatten(0, 1)[:lengths[i]].float()
        vv = vpool[tables[i]].flatten(0, 1)[:lengths[i]].float()
        want.append(plain.attention(q[i:i + 1].float(), kk, vv, torch.tensor([lengths[i] - 1]))[0])
    keys = kpool.permute(0, 2, 1, 3).contiguous().to(device)              # [pages, kv, page, d]
    values = vpool.permute(0, 2, 3, 1).contiguous().to(device).reshape(8, 2, page, dim)   # stored [pages, kv, d, page]
    table = torch.tensor([[3, 1, 6], [4, 7, -1]], dtype=torch.int32, device=device)
    out = torch.empty(2, 8 * dim, dtype=dtype, device=device)
    ops.attn_decode(q.reshape(2, -1).to(device), keys, values, table,
                    torch.tensor([0, 1, 2], dtype=torch.int32, device=device),
                    torch.tensor(lengths, dtype=torch.int32, device=device), 0, 2, out, 8, 2, dim, dim ** -0.5)
    torch.testing.assert_close(out.float().cpu().reshape(2, 8, dim), torch.stack(want),
                               atol=.015 if dtype == torch.bfloat16 else 3e-5, rtol=.02 if dtype == torch.bfloat16 else 3e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,page", [(4, 2, 16, 16), (6, 1, 32, 8), (28, 4, 128, 16), (5, 5, 48, 4),
                                                          (4, 2, 32, 12), (6, 3, 64, 24), (2, 1, 128, 48)])
@pytest.mark.parametrize("window", [0, 9])
def test_attn_prefill_portions(ops, device, dtype, heads, kv_heads, head_dim, page, window):
    """Portions of prompts at any offset: the query rows are the LAST q_len positions of kv_len keys."""
    cases = [(5, 5), (17, 3), (33, 33), (70, 2), (130, 64), (40, 1)]       # (kv_len, q_len)
    torch.manual_seed(11)
    lengths = [c[0] for c in cases]
    k = [torch.randn(n, kv_heads, head_dim).to(dtype).float() for n in lengths]
    v = [torch.randn(n, kv_heads, head_dim).to(dtype).float() for n in lengths]
    keys, values, table = build_paged(k, v, lengths, page, 64 * 16 // page, device, dtype, seed=3)
    total_q = sum(c[1] for c in cases)
    q = torch.randn(total_q, heads, head_dim).to(dtype)
    q_start, want, row = [0], [], 0
    for (n, ql), kk, vv in zip(cases, k, v):
        pos = torch.arange(n - ql, n)
        want.append(plain.attention(q[row:row + ql].float(), kk, vv, pos, window=window or None))
        row += ql
        q_start.append(row)
    want = torch.cat(want)
    # q lives inside a wider qkv buffer
    buf = torch.zeros(total_q, (heads + 2 * kv_heads) * head_dim, dtype=dtype, device=device)
    buf[:, :heads * head_dim] = q.reshape(total_q, -1).to(device)
    # also with every tile's keys cut into chunks of 32 or 64 for separate workgroups, and with tiles of 64
    # and of 128 rows (fast kernel only)
    for generic, chunk, tile_rows in ((False, 0, 0), (True, 0, 0), (False, 32, 64), (False, 64, 128), (False, 0, 64),
                                      (False, 0, 128)):
        out = torch.full((total_q, heads * head_dim), float("nan"), dtype=dtype, device=device)
        split = (math.ceil((max(lengths) + 31) / chunk) + 1 if chunk else 1, chunk, tile_rows)
        ws = torch.full((ops.attn_prefill_workspace_floats(total_q, heads, head_dim, split[0]),), float("nan"),
                        device=device) if chunk else None
        ops.attn_prefill(buf, keys, values, table, torch.tensor(q_start, dtype=torch.int32, device=device),
                         torch.tensor(lengths, dtype=torch.int32, device=device), 0, len(cases), max(c[1] for c in cases),
                         out, heads, kv_heads, head_dim, head_dim ** -0.5, window=window, generic=generic,
                         split=split, workspace=ws)
        torch.testing.assert_close(out.float().cpu().reshape(total_q, heads, head_dim), want, **ATTN_TOL[dtype])
    # the decode kernel on the one-token sequence must agree with the prefill kernel
    s = len(cases) - 1
    out1 = torch.full_like(out, float("nan"))
    ops.attn_decode(buf, keys, values, table, torch.tensor(q_start, dtype=torch.int32, device=device),
                    torch.tensor(lengths, dtype=torch.int32, device=device), s, 1, out1, heads, kv_heads, head_dim,
                    head_dim ** -0.5, window=window)
    torch.testing.assert_close(out1[q_start[s]].float().cpu().reshape(heads, head_dim), want[q_start[s]], **ATTN_TOL[dtype])


def test_attn_far_key_among_hundreds(ops, device):
    """One far key is made to dominate: a kernel that drops or misplaces it fails by O(1)."""
    heads, kv_heads, d, page, n = 4, 1, 32, 16, 700
    torch.manual_seed(3)
    k = torch.randn(n, kv_heads, d) * 0.1
    v = torch.randn(n, kv_heads, d)
    q = torch.randn(1, heads, d) * 0.1
    far = 37
    k[far, 0] = q[0, 2] / q[0, 2].norm() * 40.0          # head 2 sees key 37 almost alone
    q[0, 2] = q[0, 2] / q[0, 2].norm() * 8.0
    keys, values, table = build_paged([k], [v], [n], page, 64, device, torch.float32, seed=9)
    want = plain.attention(q, k, v, torch.tensor([n - 1]))
    assert (want[0, 2] - v[far, 0]).abs().max() < 1e-3
    for splits in (1, 3):
        out = torch.empty(1, heads * d, device=device)
        ws = torch.empty(max(1, ops.attn_decode_workspace_floats(1, heads, d, splits)), device=device)
        ops.attn_decode(q.reshape(1, -1).to(device), keys, values, table, torch.tensor([0, 1], dtype=torch.int32, device=device),
                        torch.tensor([n], dtype=torch.int32, device=device), 0, 1, out, heads, kv_heads, d, d ** -0.5,
                        splits=splits, workspace=ws)
        torch.testing.assert_close(out.cpu().reshape(1, heads, d), want, atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page,window,n,q_len", [(16, 0, 300, 48), (8, 0, 300, 48), (64, 0, 300, 48), (16, 70, 300, 48),
                                                 (4, 33, 300, 48), (12, 0, 300, 48), (24, 70, 300, 48), (48, 0, 300, 48),
                                                 (20, 33, 300, 48),
                                                 # many blocks a tile, so that the fast kernel's main loop runs, with
                                                 # and without a window that begins inside a block
                                                 (16, 0, 1000, 130), (16, 403, 1000, 130), (64, 530, 1000, 70)])
def test_attn_sharp_keys_at_edges(ops, device, dtype, page, window, n, q_len):
    """Each head's query points at ONE key that sits on an edge (of a page, of a 32-key block, of a split,
    of the window, of the sequence): a kernel that drops, doubles or misplaces that key is wrong by O(1),
    also in bfloat16, where random keys would hide it in the tolerance."""
    d = 64
    targets = [0, 1, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 127, 128, 159, 160, 255, 256, n - q_len - 1, n - q_len,
               n - 2, n - 1]
    if window:
        targets += [n - window - 1, n - window, n - window + 1, n - q_len - window, n - q_len - window + 1]
    heads = len(targets)
    gen = torch.Generator().manual_seed(77)
    unit = torch.nn.functional.normalize(torch.randn(heads, d, generator=gen), dim=1)
    k = (torch.randn(n, 1, d, generator=gen) * 0.1)
    v = torch.randn(n, 1, d, generator=gen)
    for h, p in enumerate(targets):
        k[p, 0] = unit[h] * 30.0
    k, v = k.to(dtype).float(), v.to(dtype).float()
    q_one = (unit * 8.0).to(dtype)                                     # score of the target: 30, of the rest: ~0
    keys, values, table = build_paged([k], [v], [n], page, max(320, n + 20) // page + 8, device, dtype, seed=21)
    kv_len = torch.tensor([n], dtype=torch.int32, device=device)
    # decode: the last position asks
    want = plain.attention(q_one[None].float(), k, v, torch.tensor([n - 1]), window=window or None)
    seen = [h for h, p in enumerate(targets) if not window or p > n - 1 - window]
    assert all((want[0, h] - v[targets[h], 0]).abs().max() < 2e-2 for h in seen)    # the vectors do what they are for
    q_start = torch.tensor([0, 1], dtype=torch.int32, device=device)
    for splits, generic in ((1, False), (2, False), (3, False), (7, False), (1, True), (4, True)):
        out = torch.full((1, heads * d), float("nan"), dtype=dtype, device=device)
        ws = torch.empty(max(1, ops.attn_decode_workspace_floats(1, heads, d, splits)), device=device)
        ops.attn_decode(q_one.reshape(1, -1).to(device), keys, values, table, q_start, kv_len, 0, 1, out, heads, 1, d,
                        d ** -0.5, window=window, splits=splits, workspace=ws, generic=generic)
        torch.testing.assert_close(out.float().cpu().reshape(1, heads, d), want, **ATTN_TOL[dtype])
    # prefill: the last q_len positions ask the same questions; early rows do not see late keys
    q = q_one[None].expand(q_len, heads, d).contiguous()
    want = plain.attention(q.float(), k, v, torch.arange(n - q_len, n), window=window or None)
    q_start = torch.tensor([0, q_len], dtype=torch.int32, device=device)
    ways = [(False, 0, 64), (False, 0, 128), (True, 0, 0), (False, 32, 128), (False, 96, 64)]
    if n >= 1000:                          # chunks long enough for the fast kernel's main loop, merged afterwards
        ways += [(False, 512, 128), (False, 384, 64)]
    for generic, chunk, tile_rows in ways:
        out = torch.full((q_len, heads * d), float("nan"), dtype=dtype, device=device)
        split = (math.ceil((n + 31) / chunk) + 1 if chunk else 1, chunk, tile_rows)
        ws = torch.full((ops.attn_prefill_workspace_floats(q_len, heads, d, split[0]),), float("nan"),
                        device=device) if chunk else None
        ops.attn_prefill(q.reshape(q_len, -1).to(device), keys, values, table, q_start, kv_len, 0, 1, q_len, out, heads, 1,
                         d, d ** -0.5, window=window, generic=generic, split=split, workspace=ws)
        torch.testing.assert_close(out.float().cpu().reshape(q_len, heads, d), want, **ATTN_TOL[dtype])


def test_attn_prefill_random_shapes_with_long_key_ranges(ops, device):
    """Two dozen random launches of the bfloat16 prompt attention (head sizes, groups, page sizes, one to three
    sequences of up to 2,500 keys, whole prompts and portions, windows, both tile sizes, tiles cut into chunks
    where the launcher would) against the plain implementation: the fast kernel's main loop runs from six
    32-key blocks a tile on, which the small cases above hardly reach."""
    import random
    rng = random.Random(7)
    dtype = torch.bfloat16
    for case in range(24):
        d = rng.choice([64, 128, 128, 128, 96, 256])
        kvh = rng.choice([1, 2, 4])
        heads = kvh * rng.choice([1, 2, 4, 7])
        page = rng.choice([8, 16, 16, 32, 64, 12, 48])
        lengths, qlens = [], []
        for _ in range(rng.choice([1, 1, 2, 3])):
            n = rng.choice([rng.randint(200, 700), rng.randint(700, 2500), rng.randint(33, 200)])
            lengths.append(n)
            qlens.append(rng.choice([n, rng.randint(1, min(n, 300)), rng.randint(1, n)]))
        window = rng.choice([0, 0, 0, rng.randint(40, 900)])
        gen = torch.Generator().manual_seed(case)
        k = [(torch.randn(n, kvh, d, generator=gen) * 0.7).to(dtype).float() for n in lengths]
        v = [torch.randn(n, kvh, d, generator=gen).to(dtype).float() for n in lengths]
        keys, values, table = build_paged(k, v, lengths, page, sum(math.ceil(n / page) for n in lengths) + 5, device,
                                          dtype, seed=case)
        total_q = sum(qlens)
        q = (torch.randn(total_q, heads, d, generator=gen) * 1.5).to(dtype)
        want, q_start, row = [], [0], 0
        for n, ql, kk, vv in zip(lengths, qlens, k, v):
            want.append(plain.attention(q[row:row + ql].float(), kk, vv, torch.arange(n - ql, n), window=window or None))
            row += ql
            q_start.append(row)
        buf = torch.zeros(total_q, (heads + 2 * kvh) * d, dtype=dtype, device=device)
        buf[:, :heads * d] = q.reshape(total_q, -1).to(device)
        out = torch.full((total_q, heads * d), float("nan"), dtype=dtype, device=device)
        split = ops.attn_prefill_split(len(lengths), heads, kvh, max(qlens), max(lengths), tile_rows=rng.choice([0, 0, 64, 128]))
        ws = torch.full((max(1, ops.attn_prefill_workspace_floats(total_q, heads, d, split[0])),), float("nan"), device=device)
        ops.attn_prefill(buf, keys, values, table, torch.tensor(q_start, dtype=torch.int32, device=device),
                         torch.tensor(lengths, dtype=torch.int32, device=device), 0, len(lengths), max(qlens), out, heads,
                         kvh, d, d ** -0.5, window=window, split=split, workspace=ws)
        torch.testing.assert_close(out.float().cpu().reshape(total_q, heads, d), torch.cat(want), **ATTN_TOL[dtype],
                                   msg=lambda m: f"case {case}: d {d} heads {heads}/{kvh} page {page} lengths {lengths} "
                                                 f"q {qlens} window {window} split {split}: {m}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_soft_capped_scores(ops, device, dtype):
    """softcap * tanh(score / softcap) before the softmax, decode and prompt portions, against the formula in
    torch. Queries are long enough that uncapped scores reach several times the cap: without the cap, or with
    the cap before the scale, the result is wrong by O(1)."""
    heads, kv_heads, d, page, n, q_len, cap = 4, 2, 32, 8, 75, 9, 5.0
    gen = torch.Generator().manual_seed(8)
    k = torch.randn(n, kv_heads, d, generator=gen).to(dtype).float()
    v = torch.randn(n, kv_heads, d, generator=gen).to(dtype).float()
    q = (torch.randn(q_len, heads, d, generator=gen) * 6.0).to(dtype)
    pos = torch.arange(n - q_len, n)
    kk = k.repeat_interleave(heads // kv_heads, 1)
    vv = v.repeat_interleave(heads // kv_heads, 1)
    scores = torch.einsum("qhd,khd->hqk", q.float(), kk) * d ** -0.5
    assert scores.abs().max() > 3 * cap
    capped = cap * torch.tanh(scores / cap)
    capped = capped.masked_fill(torch.arange(n)[None, None, :] > pos[None, :, None], float("-inf"))
    want = torch.einsum("hqk,khd->qhd", torch.softmax(capped, -1), vv)
    uncapped = torch.einsum("hqk,khd->qhd", torch.softmax(scores.masked_fill(
        torch.arange(n)[None, None, :] > pos[None, :, None], float("-inf")), -1), vv)
    assert (want - uncapped).abs().max() > 0.1                             # the cap matters here
    keys, values, table = build_paged([k], [v], [n], page, n // page + 3, device, dtype, seed=2)
    kv_len = torch.tensor([n], dtype=torch.int32, device=device)
    out = torch.full((q_len, heads * d), float("nan"), dtype=dtype, device=device)
    ops.attn_prefill(q.reshape(q_len, -1).to(device), keys, values, table,
                     torch.tensor([0, q_len], dtype=torch.int32, device=device), kv_len, 0, 1, q_len, out, heads,
                     kv_heads, d, d ** -0.5, softcap=cap)
    torch.testing.assert_close(out.float().cpu().reshape(q_len, heads, d), want, **ATTN_TOL[dtype])
    for splits in (1, 3):
        out1 = torch.full((1, heads * d), float("nan"), dtype=dtype, device=device)
        ws = torch.empty(max(1, ops.attn_decode_workspace_floats(1, heads, d, splits)), device=device)
        ops.attn_decode(q[-1:].reshape(1, -1).to(device), keys, values, table,
                        torch.tensor([0, 1], dtype=torch.int32, device=device), kv_len, 0, 1, out1, heads, kv_heads, d,
                        d ** -0.5, splits=splits, workspace=ws, softcap=cap)
        torch.testing.assert_close(out1.float().cpu().reshape(heads, d), want[-1], **ATTN_TOL[dtype])


@pytest.mark.parametrize("head_dim", [128, 64])
def test_attn_prefill_scores_that_keep_rising(ops, device, head_dim):
    """Scores grow from one 32-key block to the next, by a different amount per head: little (the softmax
    reference of the fast kernel stays where the first block put it and probabilities exceed 1), about as
    much as the kernel lets a score exceed its reference, and more (the reference moves and sum and output
    are rescaled, block after block). A wrong rescaling, or a reference that is moved for one of sum and
    output only, is wrong by O(1)."""
    dtype, n, q_len, page = torch.bfloat16, 448, 96, 16
    steps = [0.4, 2.0, 5.0, 5.6, 9.0, 0.0]                               # score gained per block, natural units
    heads = len(steps)
    gen = torch.Generator().manual_seed(5)
    unit = torch.nn.functional.normalize(torch.randn(head_dim, generator=gen), dim=0)
    block = (torch.arange(n) // 32).float()
    k = (unit[None] * block[:, None] + 0.02 * torch.randn(n, head_dim, generator=gen))[:, None, :]
    v = torch.randn(n, 1, head_dim, generator=gen)
    k, v = k.to(dtype).float(), v.to(dtype).float()
    q_one = torch.stack([unit * (s * head_dim ** 0.5) for s in steps]).to(dtype)       # q.k / sqrt(d) = s * block
    q = q_one[None].expand(q_len, heads, head_dim).contiguous()
    want = plain.attention(q.float(), k, v, torch.arange(n - q_len, n))
    keys, values, table = build_paged([k], [v], [n], page, n // page + 4, device, dtype, seed=4)
    kv_len = torch.tensor([n], dtype=torch.int32, device=device)
    q_start = torch.tensor([0, q_len], dtype=torch.int32, device=device)
    for generic, chunk, tile_rows in ((False, 0, 64), (False, 0, 128), (True, 0, 0), (False, 64, 128), (False, 160, 64)):
        out = torch.full((q_len, heads * head_dim), float("nan"), dtype=dtype, device=device)
        split = (math.ceil((n + 31) / chunk) + 1 if chunk else 1, chunk, tile_rows)
        ws = torch.full((ops.attn_prefill_workspace_floats(q_len, heads, head_dim, split[0]),), float("nan"),
                        device=device) if chunk else None
        ops.attn_prefill(q.reshape(q_len, -1).to(device), keys, values, table, q_start, kv_len, 0, 1, q_len, out, heads, 1,
                         head_dim, head_dim ** -0.5, generic=generic, split=split, workspace=ws)
        torch.testing.assert_close(out.float().cpu().reshape(q_len, heads, head_dim), want, **ATTN_TOL[dtype])


# ---------------------------------------------------------------------------------------
def test_sampling_greedy_ties_and_distribution(ops, device):
    vocab = 389
    logits = torch.zeros(3, vocab, device=device)
    logits[0, [5, 200, 388]] = 7.0            # tie: the lowest index wins
    logits[1, 388] = 1.0
    logits[2] = -1.0
    out = torch.empty(3, dtype=torch.int32, device=device)
    ops.sample_rows(logits, out)
    assert out.tolist() == [5, 388, 0]
    # distribution: many seeds on a small vocabulary against softmax(logits / T)
    torch.manual_seed(0)
    base = torch.randn(11) * 1.5
    rows = 20000
    temp = 0.8
    lg = base.repeat(rows, 1).to(device)
    ids = torch.empty(rows, dtype=torch.int32, device=device)
    ops.sample_rows(lg, ids, temperature=torch.full((rows,), temp, device=device),
                    seeds=torch.arange(rows, dtype=torch.int64, device=device),
                    counters=torch.zeros(rows, dtype=torch.int32, device=device))
    probs = plain.softmax_temperature(base, temp)
    counts = torch.bincount(ids.long().cpu(), minlength=11).double()
    chi2 = (((counts - rows * probs.double()) ** 2) / (rows * probs.double())).sum().item()
    assert chi2 < 40.0, chi2                   # 10 degrees of freedom: P(chi2 > 40) < 2e-5
    # same (seed, counter) -> same id whatever else is in the batch; other counters differ somewhere
    ids2 = torch.empty(5, dtype=torch.int32, device=device)
    ops.sample_rows(lg[:5], ids2, temperature=torch.full((5,), temp, device=device),
                    seeds=torch.tensor([7, 3, 7, 1, 7], dtype=torch.int64, device=device),
                    counters=torch.tensor([2, 0, 2, 0, 2], dtype=torch.int32, device=device))
    assert ids2[0] == ids2[2] == ids2[4]
    assert ids2[1].item() == ids[3].item() and ids2[3].item() == ids[1].item()
    # T -> 0+ converges to greedy
    ids3 = torch.empty(64, dtype=torch.int32, device=device)
    ops.sample_rows(lg[:64], ids3, temperature=torch.full((64,), 1e-3, device=device),
                    seeds=torch.arange(64, dtype=torch.int64, device=device),
                    counters=torch.zeros(64, dtype=torch.int32, device=device))
    assert (ids3.cpu() == int(base.argmax())).all()
    # inverse CDF with the generator's own uniform number
    u = ops.sampling_uniform(12345, 9)
    cdf = torch.cumsum(probs, 0)
    want = int((cdf > u * cdf[-1]).nonzero()[0])
    one = torch.empty(1, dtype=torch.int32, device=device)
    ops.sample_rows(lg[:1], one, temperature=torch.tensor([temp], device=device),
                    seeds=torch.tensor([12345], dtype=torch.int64, device=device),
                    counters=torch.tensor([9], dtype=torch.int32, device=device))
    assert one.item() == want
