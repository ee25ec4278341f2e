"""The argmax entry point that allocates nothing (`axk_argmax_static`), called through ctypes
as a caller without an allocator would: two calls in a row on one stream, the second with a
smaller input, each compared with `axk_argmax` on a caller's workspace; and its refusals.
"""
import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib(dtype):
    from axon_amd.kernels import build
    lib = ctypes.CDLL(build.build_kernels(dtype))
    lib.axk_last_error.restype = ctypes.c_char_p
    lib.axk_argmax.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p]
    lib.axk_argmax_static.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_void_p]
    lib.axk_argmax_workspace.argtypes = [c_int, c_int]
    lib.axk_argmax_workspace.restype = ctypes.c_long
    return lib


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_argmax_static_matches_argmax_on_two_calls_in_a_row(dtype):
    lib = _lib(dtype)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(3)
    # the second input is smaller in both directions: what the first call left in the library's
    # array lies beyond and between what the second one writes
    for rows, n, stride in [(37, 152064, 152064), (5, 4099, 4100)]:
        logits = torch.randn((rows, stride), generator=g).cuda()
        logits[0, : n // 2] = float("nan")
        logits[1, n - 1] = logits[1, :n].max()                       # equal maxima: the last index
        want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        work = torch.empty(lib.axk_argmax_workspace(rows, n) // 8, dtype=torch.int64, device="cuda")
        rc = lib.axk_argmax(c_void_p(logits.data_ptr()), stride, c_void_p(want.data_ptr()), rows, n,
                            c_void_p(work.data_ptr()), stream)
        assert rc == 0, lib.axk_last_error().decode()
        rc = lib.axk_argmax_static(c_void_p(logits.data_ptr()), stride, c_void_p(got.data_ptr()), rows, n, stream)
        assert rc == 0, lib.axk_last_error().decode()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rows, n)
        assert int(got[1]) == n - 1
        ref = torch.nan_to_num(logits[:, :n], nan=float("-inf")).cpu()
        plain = [max(range(n), key=lambda i, r=r: (float(ref[r, i]), i)) for r in (0, 2)]
        assert [int(got[0]), int(got[2])] == plain


def test_argmax_static_refuses_what_its_array_cannot_hold():
    lib = _lib("bfloat16")
    lib.axk_argmax_static_max_rows.restype = c_int
    lib.axk_argmax_static_max_n.restype = c_int
    rows, n = lib.axk_argmax_static_max_rows(), lib.axk_argmax_static_max_n()
    logits = torch.zeros((2, 64), device="cuda")
    picks = torch.zeros(2, dtype=torch.int32, device="cuda")
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    # sizes are checked before anything is launched, so the tensors need not be that large
    assert lib.axk_argmax_static(c_void_p(logits.data_ptr()), n + 1, c_void_p(picks.data_ptr()), 2, n + 1, stream) != 0
    assert b"scratch" in lib.axk_last_error()
    assert lib.axk_argmax_static(c_void_p(logits.data_ptr()), 64, c_void_p(picks.data_ptr()), rows + 1, 64, stream) != 0
    assert lib.axk_argmax_static(c_void_p(logits.data_ptr()), 64, c_void_p(picks.data_ptr()), 2, 64, stream) == 0
    torch.cuda.synchronize()
    assert picks.tolist() == [63, 63]
