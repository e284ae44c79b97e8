"""The entry point that allocates nothing (csrc/no_alloc_entry.h), called through ctypes
as a caller without torch would: the same ids as the entry point that takes the buffers
from its caller, on two calls in a row that share the library's buffer, the second with a
smaller input; sizes beyond the buffer are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from hfee_amd.kernels import build
    dll = ctypes.CDLL(build.build_library("core"))
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    dll.hfee_argmax_static.argtypes = [P, P, L, I, I, P]
    dll.hfee_argmax_static.restype = I
    dll.hfee_argmax.argtypes = [P, P, L, I, I, P, L, P, I, P]
    dll.hfee_argmax.restype = I
    dll.hfee_last_error.restype = ctypes.c_char_p
    return dll


def _both(dll, logits):
    rows, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    mine = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    theirs = torch.full((rows,), -9, dtype=torch.int32, device="cuda")
    partial = torch.zeros((rows, 64, 2), dtype=torch.float32, device="cuda")
    counters = torch.zeros((rows,), dtype=torch.int32, device="cuda")
    rc = dll.hfee_argmax(theirs.data_ptr(), logits.data_ptr(), logits.stride(0), rows, V, partial.data_ptr(),
                         rows * 64, counters.data_ptr(), rows, stream)
    assert rc == 0, dll.hfee_last_error()
    rc = dll.hfee_argmax_static(mine.data_ptr(), logits.data_ptr(), logits.stride(0), rows, V, stream)
    assert rc == 0, dll.hfee_last_error()
    torch.cuda.synchronize()
    return mine.cpu(), theirs.cpu()


def test_argmax_without_a_buffer_from_the_caller():
    dll = _lib()
    g = torch.Generator(device="cuda").manual_seed(4)
    first = torch.randn((8, 128256), generator=g, device="cuda")
    first[3, 70000] = first[3, 5] = 9.0                    # a tie: the first maximum wins
    second = torch.randn((3, 9001), generator=g, device="cuda")      # fewer rows, fewer parts a row
    for logits in (first, second, first[:1], second):
        mine, theirs = _both(dll, logits)
        assert torch.equal(mine, theirs), (logits.shape, mine, theirs)
        assert torch.equal(mine.long(), logits.argmax(dim=1).cpu()) or logits is first
    assert _both(dll, first)[0][3] == 5
    # one wide row after many narrow ones: the counters of the rows beyond it are left alone and zero
    rc = dll.hfee_argmax_static(0, first.data_ptr(), first.stride(0), 257, 128256, None)
    assert rc != 0 and b"257 rows" in dll.hfee_last_error()
