"""The entry point that allocates nothing (yalis_amd/csrc/no_alloc.h: yk_argmax_static), called
through ctypes as a caller outside this package would, against yk_argmax (caller-supplied
workspace) on the same logits: two calls in a row, the second with a smaller input, so that
what the first call left in the library's static scratch lies beside what the second wrote.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _library():
    from yalis_amd.ops.build import build_kernels

    lib = ctypes.CDLL(build_kernels("sampling"))
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.yk_last_error.restype = ctypes.c_char_p
    lib.yk_argmax_static_setup.argtypes = []
    lib.yk_argmax_static_setup.restype = ci
    lib.yk_argmax_static.argtypes = [vp, vp, ci, ci, vp]
    lib.yk_argmax_static.restype = ci
    lib.yk_argmax.argtypes = [vp, vp, ci, ci, vp, ctypes.c_size_t, vp]
    lib.yk_argmax.restype = ci
    return lib


def _logits(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((rows, vocab), generator=g)
    # ties (the lowest index must win), a row whose best is its last element, a row of -inf
    x[0, 5] = x[0, vocab - 1] = 9.0
    if rows > 1:
        x[1, vocab - 1] = 11.0
    if rows > 2:
        x[2, :] = float("-inf")
    return x.to(DEV)


def test_static_scratch_argmax_matches_the_workspace_one():
    lib = _library()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.yk_argmax_static_setup() == 0, lib.yk_last_error().decode()
    for rows, vocab, seed in ((37, 128256, 0), (5, 9001, 1)):  # the second call is the smaller one
        logits = _logits(rows, vocab, seed)
        want = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        ws = torch.empty(rows * 64, dtype=torch.float32, device=DEV)
        assert lib.yk_argmax(logits.data_ptr(), want.data_ptr(), rows, vocab, ws.data_ptr(), ws.numel(), stream) == 0
        got = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        rc = lib.yk_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream)
        assert rc == 0, lib.yk_last_error().decode()
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist()
        # and both against the plain answer, every row: torch's argmax of the host copy where a
        # row has one largest element, the lowest index among equals where it has several
        host = logits.cpu()
        plain = torch.argmax(host, dim=1).tolist()
        largest = host.max(dim=1).values
        for r in range(rows):
            ties = torch.nonzero(host[r] == largest[r]).flatten()
            assert got[r].item() == (plain[r] if ties.numel() == 1 else int(ties[0])), r
        assert got[0].item() == 5 and (rows < 3 or got[2].item() == 0)


def test_small_vocabulary_and_limits():
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    # fewer elements than slices: most slices are empty
    logits = _logits(3, 19, 2)
    got = torch.full((3,), -1, dtype=torch.int32, device=DEV)
    assert lib.yk_argmax_static(logits.data_ptr(), got.data_ptr(), 3, 19, stream) == 0, lib.yk_last_error().decode()
    torch.cuda.synchronize()
    assert got.tolist() == [5, 18, 0]
    # beyond the stated maximum: refused, nothing launched, the output untouched
    before = got.clone()
    assert lib.yk_argmax_static(logits.data_ptr(), got.data_ptr(), 1025, 19, stream) != 0
    assert b"1024" in lib.yk_last_error()
    torch.cuda.synchronize()
    assert got.tolist() == before.tolist()
    assert lib.yk_argmax_static(logits.data_ptr(), got.data_ptr(), 0, 19, stream) == 0
