"""The entry point that allocates nothing (csrc/no_alloc.h): `mlr_sample_static`, called through ctypes,
against `mlr_sample` with workspace arguments, on two calls in a row, the second with a smaller input (the
static scratch memory still holds the first call's words then)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 256
TOO_MANY_ROWS = -3


def library():
    from mini_llm_runtime_amd.kernels import build
    lib = build.load("sampling")
    ptr, c_int = ctypes.c_void_p, ctypes.c_int
    lib.mlr_sample.argtypes = [ptr, c_int, c_int, ptr, ptr, ptr, ptr, ptr, ptr, c_int, ptr]
    lib.mlr_sample_static.argtypes = [ptr, c_int, c_int, ptr, ptr, ptr, ptr, c_int, ptr]
    lib.mlr_sample.restype = lib.mlr_sample_static.restype = c_int
    return lib


def inputs(rows, vocab, seed, bad_row=None):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn((rows, vocab), generator=g) * 3).cuda()
    if bad_row is not None:
        logits[bad_row, vocab // 2] = float("inf")
    temperature = torch.where(torch.arange(rows) % 3 == 0, torch.zeros(rows), torch.full((rows,), 0.8)).cuda()
    uniform = torch.rand(rows, generator=g).cuda()
    return logits, temperature, uniform


def run_both(lib, logits, temperature, uniform):
    rows, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    out = []
    # with workspace arguments (the existing entry point)
    tokens = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    status = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    scratch_f = torch.empty(rows * (2 * 64 + 1), dtype=torch.float32, device="cuda")
    scratch_i = torch.empty(rows * 2 * 64, dtype=torch.int32, device="cuda")
    assert lib.mlr_sample(p(logits), rows, vocab, p(temperature), p(uniform), p(tokens), p(status), p(scratch_f),
                          p(scratch_i), 1, stream) == 0
    out.append((tokens.cpu().tolist(), status.cpu().tolist()))
    # without: nothing may be allocated on the device by the call
    tokens2 = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    status2 = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert lib.mlr_sample_static(p(logits), rows, vocab, p(temperature), p(uniform), p(tokens2), p(status2), 1,
                                 stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    out.append((tokens2.cpu().tolist(), status2.cpu().tolist()))
    return out


def test_static_scratch_gives_what_workspace_arguments_give():
    lib = library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.mlr_sample_static(None, 0, 0, None, None, None, None, 0, stream) == 0        # the set-up call
    # first call: the most rows the scratch memory holds, a vocabulary that is no multiple of anything
    first = run_both(lib, *inputs(MAX_ROWS, 5003, seed=1, bad_row=17))
    assert first[0] == first[1]
    assert first[0][1] == [1, 17] and first[0][0][17] == -1 and min(t for i, t in enumerate(first[0][0]) if i != 17) >= 0
    # second call, smaller in both extents: stale words of the first call lie behind and between its own
    second = run_both(lib, *inputs(5, 311, seed=2))
    assert second[0] == second[1]
    assert second[0][1] == [0, 0x7fffffff] and all(0 <= t < 311 for t in second[0][0])
    # greedy rows are the argmax with ties to the lowest id
    logits, temperature, uniform = inputs(5, 311, seed=2)
    for r in (0, 3):
        assert second[1][0][r] == int(torch.argmax(logits[r]).item())
    # a third call: one row, one token
    third = run_both(lib, *inputs(1, 1, seed=3))
    assert third[0] == third[1] == ([0], [0, 0x7fffffff])


def test_more_rows_than_the_scratch_holds_are_refused():
    lib = library()
    logits, temperature, uniform = inputs(MAX_ROWS + 1, 64, seed=4)
    tokens = torch.full((MAX_ROWS + 1,), -7, dtype=torch.int32, device="cuda")
    status = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.mlr_sample_static(p(logits), MAX_ROWS + 1, 64, p(temperature), p(uniform), p(tokens), p(status), 1, stream)
    assert rc == TOO_MANY_ROWS
    torch.cuda.synchronize()
    assert tokens.cpu().tolist() == [-7] * (MAX_ROWS + 1) and status.cpu().tolist() == [-7, -7]     # nothing ran
    assert lib.mlr_sample_static(p(logits), 4, 0, p(temperature), p(uniform), p(tokens), p(status), 1, stream) == -1
