"""The argmax entry point that allocates nothing (its partial results go through an array of the
library's own): called through ctypes, twice in a row -- the second time with a smaller input, so
that what the first call left in the array lies beside what the second writes -- and compared with
the entry point that takes a workspace."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_argmax_without_allocation_matches_the_one_with_a_workspace():
    from bare_cuda_4gib_amd.csrc import library, ops
    lib = library.load()
    lib.bc4g_argmax_static_max_rows.restype = ctypes.c_int
    lib.bc4g_argmax_static_max_rows.argtypes = []
    most = lib.bc4g_argmax_static_max_rows()
    assert most == 1024
    torch.cuda.set_device(0)
    stream = torch._C._cuda_getCurrentRawStream(0)
    g = torch.Generator().manual_seed(5)
    first = torch.randn(37, 32000, generator=g)
    first[3, 7] = first[3, 31999] = first[3, 500] = 9.0            # a tie: the lowest index
    first[4, 31999] = 11.0                                          # the maximum in the last place
    second = torch.randn(5, 301, generator=g)                       # fewer rows, a smaller and odd vocabulary
    second[0, 300] = second[0, 12] = 8.0
    for logits in (first, second):                                  # two calls in a row on the same array
        dev = logits.to(DEV).contiguous()
        out = torch.full((dev.shape[0],), -7, dtype=torch.int32, device=DEV)
        want = ops.argmax(dev)                                      # the existing entry point (workspace from torch)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        status = lib.bc4g_argmax_static(dev.data_ptr(), out.data_ptr(), dev.shape[0], dev.shape[1], stream)
        assert status == 0, lib.bc4g_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(out, want)
        assert torch.equal(out.cpu().long(), torch.stack([(row == row.max()).nonzero()[0, 0] for row in logits]))
    # the most rows it takes, and one more
    big = torch.randn(most, 130, generator=g).to(DEV)
    out = torch.empty(most, dtype=torch.int32, device=DEV)
    assert lib.bc4g_argmax_static(big.data_ptr(), out.data_ptr(), most, 130, stream) == 0
    assert torch.equal(out, ops.argmax(big))
    status = lib.bc4g_argmax_static(big.data_ptr(), out.data_ptr(), most + 1, 130, stream)
    assert status != 0 and "1024" in lib.bc4g_last_error().decode() and "1025" in lib.bc4g_last_error().decode()
