"""The greedy choice that allocates nothing (``soc_argmax_static``), called through ctypes
as a caller without torch's allocator would, against the entry point with a caller's
workspace (``soc_argmax``): two calls in a row, the second on a smaller input, so that what
the first call left in the static array must not leak into the second."""

import ctypes
from ctypes import c_char_p, c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from socrates_amd.kernels.build import load_library
    lib = load_library("sampling")
    lib.soc_argmax.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]
    lib.soc_argmax.restype = c_int
    lib.soc_argmax_static.argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p, c_char_p, c_int]
    lib.soc_argmax_static.restype = c_int
    lib.soc_argmax_static_init.argtypes = [c_char_p, c_int]
    lib.soc_argmax_static_init.restype = c_int
    return lib


def _both(lib, logits):
    n, V = logits.shape
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    n_chunks = max(1, min(64, V // 2048))
    partial = torch.empty((n, n_chunks, 2), dtype=torch.float32, device=logits.device)
    want = torch.full((n,), -1, dtype=torch.int32, device=logits.device)
    got = torch.full((n,), -1, dtype=torch.int32, device=logits.device)
    assert lib.soc_argmax(c_void_p(logits.data_ptr()), c_void_p(partial.data_ptr()), c_void_p(want.data_ptr()),
                          n, V, n_chunks, stream) == 0
    message = ctypes.create_string_buffer(256)
    err = lib.soc_argmax_static(c_void_p(logits.data_ptr()), c_void_p(got.data_ptr()), n, V, stream, message, 256)
    assert err == 0, message.value.decode()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_static_argmax_equals_workspace_argmax_on_two_calls():
    lib = _library()
    message = ctypes.create_string_buffer(256)
    assert lib.soc_argmax_static_init(message, 256) == 0, message.value.decode()
    g = torch.Generator().manual_seed(5)
    # many chunks and rows first, so that the array is full of large values and indices
    big = (torch.randn((37, 151936), generator=g) + 50.0).cuda()
    big[3, 151935] = 1e4                     # the last entry of the last chunk
    big[4, 77] = big[4, 70000] = 2e4         # equal maxima: the lowest index wins
    got, want = _both(lib, big)
    assert torch.equal(got, want)
    assert torch.equal(got.long(), big.cpu().argmax(-1))
    assert int(got[3]) == 151935 and int(got[4]) == 77
    # then fewer rows, a smaller vocabulary (fewer chunks) and values far below the first call's
    small = (torch.randn((5, 5000), generator=g) - 50.0).cuda()
    got, want = _both(lib, small)
    assert torch.equal(got, want)
    assert torch.equal(got.long(), small.cpu().argmax(-1))


def test_static_argmax_refuses_more_rows_than_it_holds():
    lib = _library()
    logits = torch.zeros((257, 8), dtype=torch.float32, device="cuda")
    out = torch.zeros((257,), dtype=torch.int32, device="cuda")
    message = ctypes.create_string_buffer(256)
    err = lib.soc_argmax_static(c_void_p(logits.data_ptr()), c_void_p(out.data_ptr()), 257, 8,
                                c_void_p(torch.cuda.current_stream().cuda_stream), message, 256)
    assert err != 0
    assert b"257" in message.value and b"256" in message.value
