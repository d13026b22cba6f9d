"""
The entry point that allocates nothing (rtn_native_lstm2_fwd_static: scratch in a fixed device array inside the
library) against rtn_native_lstm2_fwd with a caller workspace: same arguments, same results bit for bit, on two
calls in a row, the second on a smaller problem (the array keeps the first call's contents).
"""

from __future__ import annotations

import numpy
import pytest
import torch

from returnn_amd import lib

from _gpu_util import announce, get_op, random_problem, run_raw, to_dev

pytestmark = pytest.mark.gpu


def _run_static(X, W, y0, c0, i, start, step, dtype, mode):
    get_op()
    cabi = lib.load()
    Xd, Wd, y0d = (to_dev(a, dtype) for a in (X, W, y0))
    c0d, id_ = (to_dev(a, "f32") for a in (c0, i))
    T, B = i.shape
    n = y0.shape[1]
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    Y = torch.full((T, B, n), float("nan"), dtype=act, device="cuda:0")
    C = torch.full((T, B, n), float("nan"), dtype=torch.float32, device="cuda:0")
    H = torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0")
    d = torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    allocated = torch.cuda.memory_allocated()
    rc = cabi.rtn_native_lstm2_fwd_static(
        Xd.data_ptr(), Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), start, step,
        Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr(), T, B, n, dt, lib.MODES[mode], stream,
    )  # fmt: skip
    assert torch.cuda.memory_allocated() == allocated
    torch.cuda.synchronize()
    return rc, tuple(t.float().cpu().numpy() for t in (Y, C, H, d))


@pytest.mark.parametrize(
    "dtype,mode,first,second",
    [
        ("bf16", "auto", (24, 32, 1024), (9, 5, 256)),       # the benchmark's width, then a smaller problem
        ("f32", "auto", (20, 16, 512), (7, 3, 64)),
        ("f32", "stepwise", (6, 4, 96), (3, 2, 32)),          # plain per-step launches
        ("f32", "auto", (5, 3, 24), (4, 2, 7)),               # element-wise kernels (widths below 32)
    ],
)
def test_static_entry_equals_the_workspace_entry_twice(dtype, mode, first, second):
    for k, (T, B, n) in enumerate((first, second)):
        announce("static entry", dtype, mode, "call", k, "T=%i B=%i n=%i" % (T, B, n))
        X, W, y0, c0, i = random_problem(40 + k, T, B, n)
        start, step = (0, 1) if k == 0 else (1, -1)
        rc_ref, status, want = run_raw(X, W, y0, c0, i, start, step, dtype=dtype, mode=mode)
        assert rc_ref == lib.RTN_OK and status == lib.RTN_OK, lib.last_error()
        rc, got = _run_static(X, W, y0, c0, i, start, step, dtype, mode)
        assert rc == lib.RTN_OK, lib.last_error()
        for name, a, b in zip("YCHd", got, want):
            assert numpy.isfinite(a).all(), name
            assert numpy.array_equal(a, b), "%s differs (call %i)" % (name, k)


def test_static_entry_limits():
    announce("static entry limits")
    get_op()
    cabi = lib.load()
    dummy = torch.zeros((64,), dtype=torch.float32, device="cuda:0").data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    # a workspace beyond the array: refused before anything is enqueued
    T, B, n = 4, 16, 2048
    assert lib.workspace_bytes(T, B, n, lib.DTYPE_F32, lib.MODE_AUTO) > (20 << 20)
    rc = cabi.rtn_native_lstm2_fwd_static(dummy, dummy, dummy, dummy, dummy, 0, 1, dummy, dummy, dummy, dummy, T, B, n,
                                          lib.DTYPE_F32, lib.MODE_AUTO, stream)
    assert rc == lib.RTN_ERR_WORKSPACE and "static array" in lib.last_error()
    rc = cabi.rtn_native_lstm2_fwd_static(dummy, dummy, dummy, dummy, dummy, 0, 1, dummy, dummy, dummy, dummy, 4, 2, 32,
                                          lib.DTYPE_F32, lib.MODE_GRAPH, stream)
    assert rc == lib.RTN_ERR_UNSUPPORTED
    rc = cabi.rtn_native_lstm2_fwd_static(dummy, dummy, dummy, dummy, dummy, 4, 1, dummy, dummy, dummy, dummy, 4, 2, 32,
                                          lib.DTYPE_F32, lib.MODE_AUTO, stream)
    assert rc == lib.RTN_ERR_RANGE
    torch.cuda.synchronize()
