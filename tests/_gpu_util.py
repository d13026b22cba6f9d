"""Helpers of the GPU parity tests: run the op through the C ABI on cuda:0 and bring results back as numpy."""

from __future__ import annotations

import contextlib
import os
import sys

import numpy
import torch

from returnn_amd import build, lib, native_op, torch_native_op


def get_op(mode="auto"):
    if not os.path.exists(build.LIB_PATH):
        build.build_library()
    return torch_native_op.make_op(native_op.NativeLstm2, mode=mode)


@contextlib.contextmanager
def env(**kwargs):
    """Temporarily set environment variables of the library (it reads them once and again when asked to)."""
    old = {k: os.environ.get(k) for k in kwargs}
    try:
        for k, v in kwargs.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = str(v)
        lib.reload_env()
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        lib.reload_env()


def announce(*what):
    """Name the case before any GPU work so that a fault can be traced to it."""
    print("[gpu case]", *what, flush=True)
    sys.stdout.flush()


def to_dev(a: numpy.ndarray, dtype: str):
    t = torch.from_numpy(numpy.ascontiguousarray(a, dtype=numpy.float32)).to("cuda:0")
    return t.to(torch.bfloat16) if dtype == "bf16" else t


def run_op(X, W, y0, c0, i, start=0, step=1, *, dtype="f32", mode="auto", check_status=True):
    """
    :return: Y, C, H, d, y_last as float32 numpy arrays
    """
    op = get_op(mode)
    Xd, Wd, y0d = (to_dev(a, dtype) for a in (X, W, y0))
    c0d, id_ = (to_dev(a, "f32") for a in (c0, i))
    Y, C, H, d = op(Xd, Wd, y0d, c0d, id_, start, step)
    y_last = torch_native_op.lstm_last_output(Y, y0d, id_, start, step) if i.shape[0] > 0 else y0d
    torch.cuda.synchronize()
    return tuple(t.float().cpu().numpy() for t in (Y, C, H, d, y_last))


def run_raw(X, W, y0, c0, i, start=0, step=1, *, dtype="f32", mode="auto"):
    """Direct call of the C ABI with explicit workspace; returns outputs and the status code of the run."""
    get_op()
    cabi = lib.load()
    Xd, Wd, y0d = (to_dev(a, dtype) for a in (X, W, y0))
    c0d, id_ = (to_dev(a, "f32") for a in (c0, i))
    T, B = i.shape
    n = y0.shape[1]
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    md = lib.MODES[mode]
    # poison the outputs: the library must write every element itself
    Y = torch.full((T, B, n), float("nan"), dtype=act, device="cuda:0")
    C = torch.full((T, B, n), float("nan"), dtype=torch.float32, device="cuda:0")
    H = torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0")
    d = torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda:0")
    ws = torch.empty((max(lib.workspace_bytes(T, B, n, dt, md), 256),), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    rc = cabi.rtn_native_lstm2_fwd(
        Xd.data_ptr(), Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), start, step,
        Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr(), T, B, n, dt, md, ws.data_ptr(), ws.numel(), stream,
    )  # fmt: skip
    status = cabi.rtn_native_lstm2_fwd_status(ws.data_ptr(), stream) if rc == 0 and T > 0 and B * n > 0 else rc
    torch.cuda.synchronize()
    return rc, status, tuple(t.float().cpu().numpy() for t in (Y, C, H, d))


def random_problem(seed, T, B, n, *, ragged=True, full_first=True, scale_x=0.5):
    rng = numpy.random.default_rng(seed)
    X = rng.normal(0, scale_x, (T, B, 4 * n)).astype(numpy.float32)
    W = rng.uniform(-1.0, 1.0, (n, 4 * n)).astype(numpy.float32) / numpy.float32(numpy.sqrt(max(n, 1)))
    y0 = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    c0 = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    if ragged and T > 0:
        lens = rng.integers(1, T + 1, size=(B,))
        if full_first:
            lens[0] = T
        i = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    else:
        i = numpy.ones((T, B), dtype=numpy.float32)
    return X, W, y0, c0, i


def run_multi_raw(problems, *, dtype="f32", mode="auto"):
    """
    Several op calls of one shape through ``rtn_native_lstm2_fwd_multi`` with explicit workspace and poisoned outputs.

    :param problems: ``[(X, W, y0, c0, i, start, step), ...]`` as numpy arrays, all of one shape
    :return: plan text, per call ``(Y, C, H, d, y_last)`` as float32 numpy arrays, per call the status words
        ``(status[0], status[1])`` of its workspace slice (0, 0 = no wait expired, every group of an XCD-local plan on one XCD)
    """
    get_op()
    cabi = lib.load()
    count = len(problems)
    T, B = problems[0][4].shape
    n = problems[0][2].shape[1]
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    md = lib.MODES[mode]
    plan = lib.describe_multi_plan(count, T, B, n, dt, md)
    arr = (lib.Lstm2Call * count)()
    keep, outs = [], []
    for k, (X, W, y0, c0, i, start, step) in enumerate(problems):
        Xd, Wd, y0d = (to_dev(a, dtype) for a in (X, W, y0))
        c0d, id_ = (to_dev(a, "f32") for a in (c0, i))
        Y = torch.full((T, B, n), float("nan"), dtype=act, device="cuda:0")
        C = torch.full((T, B, n), float("nan"), dtype=torch.float32, device="cuda:0")
        H = torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0")
        d = torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda:0")
        keep.append((Xd, Wd, y0d, c0d, id_))
        outs.append((Y, C, H, d, y0d, id_, start, step))
        arr[k] = lib.Lstm2Call(Xd.data_ptr(), Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), start, step,
                               Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr())  # fmt: skip
    nbytes = int(cabi.rtn_native_lstm2_fwd_multi_workspace_bytes(count, T, B, n, dt, md))
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    lib.check(cabi.rtn_native_lstm2_fwd_multi(arr, count, T, B, n, dt, md, ws.data_ptr(), ws.numel(), stream))
    lib.check(cabi.rtn_native_lstm2_fwd_multi_status(ws.data_ptr(), count, T, B, n, dt, md, stream))
    torch.cuda.synchronize()
    each = nbytes // count
    words = [tuple(int(v) for v in ws[k * each : k * each + 8].cpu().numpy().view(numpy.uint32)) for k in range(count)]
    results = []
    for Y, C, H, d, y0d, id_, start, step in outs:
        y_last = torch_native_op.lstm_last_output(Y, y0d, id_, start, step)
        results.append(tuple(t.float().cpu().numpy() for t in (Y, C, H, d, y_last)))
    return plan, results, words
