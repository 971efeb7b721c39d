"""The argmax entry point that allocates nothing (csrc/no_alloc.h), called through
ctypes the way a caller without torch would, against the ordinary entry point
``tk_argmax`` (whose scratch the caller brings).

Two calls in a row share the library's fixed scratch array; the second is smaller, so
entries that the first call left behind lie beside the ones the second call writes.
"""

import ctypes
from ctypes import c_int, c_long, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _entry_points():
    from tokamak_amd.kernels.build import load_library

    lib = load_library("sampling")
    plain = lib.tk_argmax
    plain.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p]
    plain.restype = c_int
    fixed = lib.tk_argmax_no_alloc
    fixed.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p]
    fixed.restype = c_int
    lib.tk_argmax_no_alloc_max_rows.restype = c_int
    lib.tk_argmax_segments.restype = c_int
    return lib, plain, fixed


def _logits(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, vocab, generator=g)
    x[0, vocab // 3] = x[0, vocab - 1] = 40.0        # a tie: the lower index wins
    if rows > 1:
        x[1, :] = float("nan")                       # a row without a number: token 0
    return x


def test_no_alloc_argmax_matches_the_ordinary_entry_point_twice():
    lib, plain, fixed = _entry_points()
    segments = lib.tk_argmax_segments()
    stream = c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    torch.cuda.set_device(DEV)
    for rows, vocab, seed in ((37, 151936, 0), (5, 1003, 1)):       # the second call is smaller
        x = _logits(rows, vocab, seed).to(DEV)
        want_i = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        want_v = torch.zeros(rows, dtype=torch.float32, device=DEV)
        part_v = torch.empty(rows * segments, dtype=torch.float32, device=DEV)
        part_i = torch.empty(rows * segments, dtype=torch.int32, device=DEV)
        got_i = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        got_v = torch.zeros(rows, dtype=torch.float32, device=DEV)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(DEV)
        assert plain(x.data_ptr(), want_i.data_ptr(), want_v.data_ptr(), part_v.data_ptr(), part_i.data_ptr(),
                     rows, vocab, x.stride(0), stream) == 0
        assert fixed(x.data_ptr(), got_i.data_ptr(), got_v.data_ptr(), rows, vocab, x.stride(0), stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(DEV) == before
        assert got_i.tolist() == want_i.tolist()
        assert torch.equal(got_v.cpu(), want_v.cpu())
        # and both agree with the definition: first maximum, NaN never wins
        ref = x.cpu()
        assert got_i[0].item() == vocab // 3
        if rows > 1:
            assert got_i[1].item() == 0
        assert got_i[2:].tolist() == ref[2:].argmax(-1).tolist()


def test_no_alloc_argmax_refuses_more_rows_than_its_scratch_holds():
    lib, _, fixed = _entry_points()
    limit = lib.tk_argmax_no_alloc_max_rows()
    torch.cuda.set_device(DEV)
    stream = c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    x = torch.zeros(limit + 1, 8, device=DEV)
    out = torch.full((limit + 1,), -7, dtype=torch.int32, device=DEV)
    assert fixed(x.data_ptr(), out.data_ptr(), None, limit + 1, 8, 8, stream) == -3
    torch.cuda.synchronize()
    assert (out == -7).all()                                   # nothing was launched
    assert fixed(x.data_ptr(), out.data_ptr(), None, limit, 8, 8, stream) == 0
    torch.cuda.synchronize()
    assert (out[:limit] == 0).all() and out[limit].item() == -7
