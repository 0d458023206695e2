"""`tw_sample_rows_static`, the sampler's entry point for callers that cannot allocate, called through ctypes
the way such a caller would, against `tw_sample_rows` with a workspace: two calls in a row, the second with a
smaller input (the built-in scratch memory still holds the first call's partial results then)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from tessweave_engine_amd.kernels import build
    lib = ctypes.CDLL(str(build.ensure_built()))
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    lib.tw_sample_rows.restype = I
    lib.tw_sample_rows.argtypes = [P, L, I, I, P, P, P, P, P, L, P]
    lib.tw_sample_rows_static.restype = I
    lib.tw_sample_rows_static.argtypes = [P, L, I, I, P, P, P, P, P]
    lib.tw_sample_workspace_bytes.restype = L
    lib.tw_sample_workspace_bytes.argtypes = [I]
    lib.tw_error_string.restype = ctypes.c_char_p
    lib.tw_error_string.argtypes = [I]
    return lib


def _case(rows, vocab, seed, device):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).to(device)
    logits[0, vocab // 2] = logits[0, vocab - 1] = 50.0                      # a tie for the greedy row: lowest index
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.1 * r for r in range(rows)], device=device)
    seeds = torch.arange(100, 100 + rows, dtype=torch.int64, device=device)
    counters = torch.arange(rows, dtype=torch.int32, device=device) * 7
    return logits, temperature, seeds, counters


def test_the_entry_point_that_allocates_nothing_matches_the_one_with_a_workspace(device):
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    # one call first: the look-up of the built-in array's address and the load of the kernels' code happen once
    # per device and are not what "allocates nothing" is about
    logits, temperature, seeds, counters = _case(3, 100, 9, device)
    first = torch.empty(3, dtype=torch.int32, device=device)
    assert lib.tw_sample_rows_static(logits.data_ptr(), logits.stride(0), 3, 100, temperature.data_ptr(),
                                     seeds.data_ptr(), counters.data_ptr(), first.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    for rows, vocab, seed in ((37, 152064, 1), (5, 1001, 2)):                # the second call is smaller
        logits, temperature, seeds, counters = _case(rows, vocab, seed, device)
        want = torch.full((rows,), -1, dtype=torch.int32, device=device)
        got = torch.full((rows,), -2, dtype=torch.int32, device=device)
        need = lib.tw_sample_workspace_bytes(rows)
        workspace = torch.empty(need, dtype=torch.uint8, device=device)
        args = (logits.data_ptr(), logits.stride(0), rows, vocab, temperature.data_ptr(), seeds.data_ptr(),
                counters.data_ptr())
        assert lib.tw_sample_rows(*args, want.data_ptr(), workspace.data_ptr(), need, stream) == 0
        torch.cuda.synchronize()
        # torch's counters see only torch's own allocator; the driver's count of free bytes sees a hipMalloc of
        # the library's too
        before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        free_before = torch.cuda.mem_get_info()[0]
        assert lib.tw_sample_rows_static(*args, got.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] >= free_before
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
        assert got.tolist() == want.tolist() and all(0 <= t < vocab for t in got.tolist())
        assert got[0].item() == vocab // 2
        # greedy only (no temperature, seeds or counters)
        assert lib.tw_sample_rows_static(logits.data_ptr(), logits.stride(0), rows, vocab, None, None, None,
                                         got.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert got.tolist() == logits.argmax(-1).tolist()
    # more rows than the built-in scratch memory holds: refused with a code that says so, nothing written
    rows = 257
    logits, temperature, seeds, counters = _case(rows, 64, 3, device)
    got = torch.full((rows,), -2, dtype=torch.int32, device=device)
    code = lib.tw_sample_rows_static(logits.data_ptr(), logits.stride(0), rows, 64, temperature.data_ptr(),
                                     seeds.data_ptr(), counters.data_ptr(), got.data_ptr(), stream)
    assert code != 0 and b"at most 256 rows" in lib.tw_error_string(code)
    torch.cuda.synchronize()
    assert (got == -2).all()
    # exactly the maximum is taken
    logits, temperature, seeds, counters = _case(256, 300, 4, device)
    got = torch.full((256,), -2, dtype=torch.int32, device=device)
    want = torch.full((256,), -1, dtype=torch.int32, device=device)
    need = lib.tw_sample_workspace_bytes(256)
    workspace = torch.empty(need, dtype=torch.uint8, device=device)
    args = (logits.data_ptr(), logits.stride(0), 256, 300, temperature.data_ptr(), seeds.data_ptr(), counters.data_ptr())
    assert lib.tw_sample_rows(*args, want.data_ptr(), workspace.data_ptr(), need, stream) == 0
    assert lib.tw_sample_rows_static(*args, got.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert got.tolist() == want.tolist()
