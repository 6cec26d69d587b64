"""The greedy choice through the entry point that allocates nothing (``dryft_argmax_rows_noalloc``), called
through ctypes as a caller without torch's allocator would, against the entry point with caller-owned buffers."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ENTRIES = 16384        # DRYFT_ARGMAX_NOALLOC_ENTRIES of csrc/sampling.h


def entry_point():
    from dryft_amd.csrc import build
    lib = build.load("sampling")
    fn = lib.dryft_argmax_rows_noalloc
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int,
                   ctypes.c_void_p]
    fn.restype = ctypes.c_int
    return fn


def test_argmax_without_allocation_equals_argmax_with_buffers():
    from dryft_amd.csrc import ops
    fn = entry_point()
    torch.manual_seed(3)
    stream = torch.cuda.current_stream().cuda_stream
    # one call beforehand: the library's code object is loaded and the array's address looked up, once per device
    first = torch.randn(2, 5000, device=DEV)
    assert fn(first.data_ptr(), 2, 5000, first.stride(0), torch.empty(2, dtype=torch.int32, device=DEV).data_ptr(), 2,
              stream) == 0
    torch.cuda.synchronize()
    # two calls in a row on the same array: the second is smaller and must not see what the first one left
    for rows, vocab, chunks in ((64, 151936, 64), (5, 50000, 24), (3, 300, 1)):
        logits = torch.randn(rows, vocab, device=DEV)
        logits[0, vocab - 7] = logits[0, 11] = 50.0              # equal maxima: the lowest index wins
        logits[rows - 1, vocab - 1] = 60.0                       # the last entry of the last stretch
        want = ops.argmax_rows(logits, torch.empty(rows, dtype=torch.int32, device=DEV))
        got = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
        # free device memory as the driver counts it (torch's own counters would not see a hipMalloc in the library)
        torch.cuda.synchronize()
        before = torch.cuda.mem_get_info()[0]
        rc = fn(logits.data_ptr(), rows, vocab, logits.stride(0), got.data_ptr(), chunks, stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before, "the call changed the device's free memory"
        assert torch.equal(got, want), (rows, vocab, chunks)
        assert got[0].item() == 11 and got[rows - 1].item() == vocab - 1
        assert torch.equal(got.long().cpu(), logits.argmax(-1).cpu())
    # rows whose stride is wider than the vocabulary
    wide = torch.randn(4, 9000, device=DEV)
    got = torch.empty(4, dtype=torch.int32, device=DEV)
    assert fn(wide.data_ptr(), 4, 8500, wide.stride(0), got.data_ptr(), 4, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(got.long().cpu(), wide[:, :8500].argmax(-1).cpu())


def test_argmax_without_allocation_refuses_what_does_not_fit(capfd):
    fn = entry_point()
    rows, chunks = ENTRIES // 64 + 1, 64
    logits = torch.zeros(rows, 64 * 2048, device=DEV)
    out = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert fn(logits.data_ptr(), rows, logits.shape[1], logits.stride(0), out.data_ptr(), chunks, stream) == -2
    assert "exceed the library's scratch" in capfd.readouterr().err
    torch.cuda.synchronize()
    assert (out == -7).all(), "a refused call must launch nothing"
    assert fn(logits.data_ptr(), rows - 1, logits.shape[1], logits.stride(0), out.data_ptr(), chunks, stream) == 0
    torch.cuda.synchronize()
    assert (out[:rows - 1] == 0).all()                        # all equal: index 0
    assert fn(0, 2, 100, 100, out.data_ptr(), 1, stream) == -1
    assert fn(logits.data_ptr(), 0, 100, 100, out.data_ptr(), 1, stream) == 0
