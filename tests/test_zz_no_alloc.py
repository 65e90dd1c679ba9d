"""The argmax entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a caller
that cannot allocate would, against apc_argmax_rows on the same logits."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _entry_points():
    from allpaca_amd.kernels import build
    lib = ctypes.CDLL(build.build("plain"))
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.apc_argmax_rows_no_alloc.argtypes = [P, I, I, I, P, P]
    lib.apc_argmax_rows_no_alloc.restype = I
    lib.apc_argmax_rows.argtypes = [P, I, I, I, P, P, P]
    lib.apc_argmax_rows.restype = I
    return lib


def _logits(rows, V, ld, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn((rows, ld), generator=g, dtype=torch.float32)
    # ties: the maximum appears twice in some rows, in different pieces of the row; one row has nothing above -inf
    for r in range(0, rows, 3):
        top = float(x[r, :V].max()) + 1.0
        a, b = (r * 7919) % V, (r * 104729 + V // 2) % V
        x[r, a] = top
        x[r, b] = top
    if rows > 4:
        x[4, :V] = float("-inf")
    x[:, V:] = 1e30   # beyond the row's width: must not be looked at
    return x.cuda()


def _expected(x, V):
    a = x[:, :V].cpu().numpy()
    want = a.argmax(axis=1).astype(np.int32)     # numpy takes the first maximum too
    want[np.isneginf(a.max(axis=1))] = 0
    return want


def test_no_alloc_argmax_equals_the_workspace_one_on_two_calls_in_a_row():
    lib = _entry_points()
    stream = torch.cuda.current_stream().cuda_stream
    # the second call is smaller in both directions, so it finds the first call's pieces in the array
    for rows, V, ld, seed in ((37, 128256, 128256, 1), (5, 8200, 8208, 2)):
        x = _logits(rows, V, ld, seed)
        got = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        ref = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        ws = torch.empty(2 * rows * 64, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        assert lib.apc_argmax_rows_no_alloc(x.data_ptr(), ld, rows, V, got.data_ptr(), stream) == 0
        assert lib.apc_argmax_rows(x.data_ptr(), ld, rows, V, ref.data_ptr(), ws.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), ref.cpu().numpy())
        assert np.array_equal(got.cpu().numpy(), _expected(x, V))


def test_no_alloc_argmax_narrow_rows_and_limits():
    lib = _entry_points()
    stream = torch.cuda.current_stream().cuda_stream
    x = _logits(9, 1003, 1003, 3)                 # below 8192: one block a row, no pieces
    got = torch.full((9,), -7, dtype=torch.int32, device="cuda")
    assert lib.apc_argmax_rows_no_alloc(x.data_ptr(), 1003, 9, 1003, got.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), _expected(x, 1003))
    # more rows than the array has room for: refused, nothing launched
    assert lib.apc_argmax_rows_no_alloc(x.data_ptr(), 8192, 1025, 8192, got.data_ptr(), stream) == -3
    assert lib.apc_argmax_rows_no_alloc(x.data_ptr(), 100, 2, 8192, got.data_ptr(), stream) == -1
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), _expected(x, 1003))
