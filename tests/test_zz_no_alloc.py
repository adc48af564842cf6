"""The entry point that allocates nothing (csrc/no_alloc.h), called through
ctypes as a caller without Python bindings would: its choices must equal those
of the existing argmax entry, whose scratch the caller brings, on two calls in
a row, the second with a smaller input that leaves most of the built-in scratch
holding the first call's values."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_ROWS = 256      # ALOFA_ARGMAX_NO_ALLOC_MAX_ROWS


def _lib():
    from alofa_amd.csrc.build import load
    lib = load()
    lib.alofa_argmax_no_alloc.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.alofa_argmax_no_alloc.restype = ctypes.c_int
    lib.alofa_argmax.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.alofa_argmax.restype = ctypes.c_int
    return lib


def _logits(rows, vocab, stride, seed):
    """Rows with ties: the maximum stands at several places, so the lowest index must win; what lies
    between a row's end and the next row's start is larger than any entry and must not be seen."""
    import torch
    rnd = np.random.default_rng(seed)
    x = rnd.standard_normal((rows, stride)).astype(np.float32)
    x[:, vocab:] = 100.0
    for r in range(rows):
        places = rnd.integers(0, vocab, size=3)
        x[r, places] = 7.5
    return torch.from_numpy(x).cuda(), x[:, :vocab].argmax(axis=1).astype(np.int32)


def test_no_alloc_argmax_equals_the_entry_with_a_scratch_argument():
    import torch
    lib = _lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the second call is smaller in rows and in row length than the first
    for call, (rows, vocab, stride) in enumerate([(64, 151936, 151936), (5, 9001, 9007)]):
        logits, want = _logits(rows, vocab, stride, seed=call)
        theirs = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        ours = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
        brought = torch.empty(2 * 64 * rows, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        assert lib.alofa_argmax(theirs.data_ptr(), logits.data_ptr(), stride, rows, vocab, brought.data_ptr(), stream) == 0, lib.alofa_last_error()
        # free device memory as the driver counts it (hipMemGetInfo): an allocation by the library itself would
        # show here, which torch's own counters, that see only torch's allocator, would miss
        torch.cuda.synchronize()
        before, held = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        assert lib.alofa_argmax_no_alloc(ours.data_ptr(), logits.data_ptr(), stride, rows, vocab, stream) == 0, lib.alofa_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_reserved() == held, f"call {call}: device memory was taken"
        assert np.array_equal(ours.cpu().numpy(), theirs.cpu().numpy()), f"call {call}: differs from the existing entry"
        assert np.array_equal(ours.cpu().numpy(), want), f"call {call}: differs from the first maximum"


def test_no_alloc_argmax_refuses_what_does_not_fit():
    import torch
    lib = _lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    logits = torch.zeros((MAX_ROWS + 1, 64), dtype=torch.float32, device="cuda")
    out = torch.zeros(MAX_ROWS + 1, dtype=torch.int32, device="cuda")
    assert lib.alofa_argmax_no_alloc(out.data_ptr(), logits.data_ptr(), 64, MAX_ROWS + 1, 64, stream) == 1
    assert b"at most 256 rows" in lib.alofa_last_error()
    assert lib.alofa_argmax_no_alloc(out.data_ptr(), logits.data_ptr(), 32, 4, 64, stream) == 1      # rows would overlap
    assert lib.alofa_argmax_no_alloc(None, logits.data_ptr(), 64, 4, 64, stream) == 1
    # the largest size it takes, and a row shorter than the 64 chunks
    assert lib.alofa_argmax_no_alloc(out.data_ptr(), logits.data_ptr(), 64, MAX_ROWS, 64, stream) == 0, lib.alofa_last_error()
    logits[3, 40] = 1.0
    assert lib.alofa_argmax_no_alloc(out.data_ptr(), logits.data_ptr(), 64, 4, 41, stream) == 0, lib.alofa_last_error()
    torch.cuda.synchronize()
    assert out[:4].tolist() == [0, 0, 0, 40]
