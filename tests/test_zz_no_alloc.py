"""The entry point that allocates nothing (``ts_argmax_static``, csrc/ts_no_alloc.h), called
through ``ctypes`` as a caller without torch's allocator would: its tokens equal those of the
entry point that takes a scratch buffer (``ts_argmax``) on two calls in a row, the second with
a smaller input, whatever the first call left in the library's own array."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_argmax_without_allocation_equals_argmax_with_scratch():
    from turboserve_amd.kernels import build

    lib = ctypes.CDLL(str(build.ensure_module("core")))
    static = lib.ts_argmax_static
    static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    static.restype = ctypes.c_int
    plain = lib.ts_argmax
    plain.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    plain.restype = ctypes.c_int

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    stream = torch.cuda.current_stream(device).cuda_stream
    generator = torch.Generator(device=device)
    generator.manual_seed(11)
    # Inputs and outputs of both calls exist before the first call; the calls allocate nothing.
    shapes = [(37, 5003), (5, 301)]  # the second is smaller in rows and in vocabulary
    cases = []
    for rows, vocab in shapes:
        logits = torch.randn((rows, vocab), device=device, generator=generator)
        logits[rows // 2, vocab - 1] = 50.0          # a winner in the last, shorter slice
        logits[0, 7] = logits[0, 300] = 60.0         # a tie: the lowest index wins
        cases.append((logits, torch.full((rows,), -1, dtype=torch.int32, device=device),
                      torch.full((rows,), -1, dtype=torch.int32, device=device),
                      torch.empty((rows, 128), dtype=torch.int32, device=device)))
    torch.cuda.synchronize(device)
    before = torch.cuda.memory_allocated(device)
    for logits, got, want, scratch in cases:
        rows, vocab = logits.shape
        assert static(got.data_ptr(), logits.data_ptr(), rows, vocab, stream) == 0
        assert plain(want.data_ptr(), logits.data_ptr(), scratch.data_ptr(), rows, vocab, stream) == 0
    torch.cuda.synchronize(device)
    assert torch.cuda.memory_allocated(device) == before
    for logits, got, want, _ in cases:
        assert torch.equal(got, want), (got.tolist(), want.tolist())
        assert torch.equal(got.long().cpu(), logits.argmax(dim=-1).cpu())
        assert int(got[0]) == 7 and int(got[logits.shape[0] // 2]) == logits.shape[1] - 1
    # Sizes beyond the array are refused with the shape error and launch nothing; no rows is fine.
    logits, got, _, _ = cases[0]
    assert static(got.data_ptr(), logits.data_ptr(), 1025, 4, stream) == 2
    assert static(got.data_ptr(), logits.data_ptr(), 0, 4, stream) == 0
    assert static(None, logits.data_ptr(), 3, 4, stream) == 4
    assert static(got.data_ptr(), logits.data_ptr(), 3, 0, stream) == 4
