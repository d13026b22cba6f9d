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

    def call():
        return cabi.rtn_native_lstm2_fwd_static(
            Xd.data_ptr(), Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), start, step,
            Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr(), T, B, n, dt, lib.MODES[mode], stream,
        )  # fmt: skip

    # A first call lets the runtime do what it does once per kernel (code object, symbol address); the second one is
    # the one measured: torch's allocator must not have been asked for anything, and the device's free memory must not
    # have shrunk either (an allocation inside the library would not go through torch).
    rc = call()
    torch.cuda.synchronize()
    if rc != lib.RTN_OK:
        return rc, None
    Y.fill_(float("nan")); C.fill_(float("nan")); H.fill_(float("nan")); d.fill_(float("nan"))  # noqa: E702
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    rc = call()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == allocated
    assert torch.cuda.mem_get_info()[0] >= free_before, "free device memory shrank during a call of the static entry"
    return rc, tuple(t.float().cpu().numpy() for t in (Y, C, H, d))


@pytest.mark.parametrize(
    "dtype,mode,first,second",
    [
        ("bf16", "auto", (24, 32, 1024), (9, 5, 256)),       # the benchmark's width, then a smaller problem
        ("f32", "auto", (20, 16, 512), (7, 3, 64)),
        ("f32", "stepwise", (6, 4, 96), (3, 2, 32)),          # plain per-step launches
        ("f32", "auto", (5, 3, 24), (4, 2, 7)),               # element-wise kernels (widths below 32)
        ("f32", "auto", (6, 4, 100), (3, 2, 40)),             # widths run zero-padded: the padded copies live in the array too
        ("bf16", "auto", (5, 8, 200), (4, 3, 72)),
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
