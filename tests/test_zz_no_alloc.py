"""The arg-max entry point that allocates nothing, called through ctypes, against the
entry point that takes a workspace: two calls in a row on one GPU, the second with a
smaller input, so that what the first call left in the library's own array would show
if the second read it."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 256  # RV_NO_ALLOC_MAX_ROWS of csrc/no_alloc.h


def _library():
    from rvllm_amd.kernels import ops

    lib = ops.library()
    lib.rv_argmax_no_alloc.restype = ctypes.c_int
    lib.rv_no_alloc_init.restype = ctypes.c_int
    lib.rv_no_alloc_init.argtypes = []
    lib.rv_argmax_no_alloc.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                       ctypes.c_longlong, ctypes.c_void_p]
    return lib


def _call(lib, logits, out):
    rows, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return lib.rv_argmax_no_alloc(stream, ctypes.c_void_p(logits.data_ptr()), rows, vocab, logits.stride(0),
                                  ctypes.c_void_p(out.data_ptr()))


def _logits(rows, vocab, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn((rows, vocab), generator=g)
    for r in range(rows):  # equal maxima (the lowest id wins) and NaN (skipped) in every row
        top = x[r].max() + 1.0
        ids = torch.randint(0, vocab, (3,), generator=g)
        x[r, ids] = top
        x[r, torch.randint(0, vocab, (2,), generator=g)] = float("nan")
    return x.cuda()


def test_argmax_no_alloc_equals_argmax_on_two_calls_in_a_row():
    from rvllm_amd.kernels import ops

    lib = _library()
    torch.cuda.set_device(0)
    big = _logits(8, 262208, seed=0)
    small = _logits(3, 509, seed=1)
    out_big = torch.full((8,), -7, dtype=torch.int32, device="cuda")
    out_small = torch.full((3,), -7, dtype=torch.int32, device="cuda")
    want_big = ops.argmax(big)
    want_small = ops.argmax(small)
    torch.cuda.synchronize()

    # the set-up call, once per device and outside any capture: after it not even the first call looks anything up
    assert lib.rv_no_alloc_init() == 0, lib.rv_last_error().decode()
    assert lib.rv_no_alloc_init() == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert _call(lib, big, out_big) == 0, lib.rv_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # the first call took no device memory
    assert _call(lib, small, out_small) == 0, lib.rv_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # nor did the second
    assert torch.equal(out_big, want_big)
    assert torch.equal(out_small, want_small)
    # and against the definition: the lowest id among the largest values that are no NaN
    for x, got in ((big, out_big), (small, out_small)):
        clean = torch.where(torch.isnan(x), torch.full_like(x, float("-inf")), x)
        first = (clean == clean.max(dim=1, keepdim=True).values).int().argmax(dim=1)
        assert torch.equal(got.long(), first)


def test_argmax_no_alloc_refuses_more_rows_than_its_array_holds():
    lib = _library()
    torch.cuda.set_device(0)
    x = torch.zeros((MAX_ROWS + 1, 16), device="cuda")
    out = torch.full((MAX_ROWS + 1,), -7, dtype=torch.int32, device="cuda")
    assert _call(lib, x, out) != 0
    assert "rows" in lib.rv_last_error().decode()
    torch.cuda.synchronize()
    assert bool((out == -7).all())  # nothing ran
    full = torch.randn((MAX_ROWS, 700), device="cuda")
    out = torch.empty(MAX_ROWS, dtype=torch.int32, device="cuda")
    assert _call(lib, full, out) == 0, lib.rv_last_error().decode()
    assert torch.equal(out.long(), full.argmax(dim=1))
