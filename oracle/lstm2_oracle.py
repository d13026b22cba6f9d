"""
ctypes binding of the C oracle in ``oracle/lstm2_oracle.c`` -- test infrastructure only.

The C file restates the reference op (returnn/native_op.py:1081-1121, :1184-1285;
returnn/native_op.cpp:1032-1067) and is the checker for the HIP path and the timed
CPU baseline.  It is never the product: nothing under ``returnn_amd/`` imports it.

Every function here is pinned by tests against golden vectors, closed forms, finite differences or autograd
(tests/test_oracle*.py), with one exception stated where it applies: ``lstm_low_mem_bwd`` on masks with holes is a
literal restatement of the reference's formulas -- parity unpinned there.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Tuple

import numpy

_dir = os.path.dirname(os.path.abspath(__file__))
_so = os.path.join(_dir, "liblstm2_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile next to it. Returns the path of the library."""
    if force and os.path.exists(_so):
        os.remove(_so)
    subprocess.check_call(["make", "-s", "-C", _dir])
    return _so


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_so):
            build()
        lib = ctypes.CDLL(_so)
        for suffix, ptr in (("f32", ctypes.POINTER(ctypes.c_float)), ("f64", ctypes.POINTER(ctypes.c_double))):
            fwd = getattr(lib, "lstm2_oracle_fwd_" + suffix)
            fwd.restype = ctypes.c_int
            fwd.argtypes = [ptr] * 5 + [ctypes.c_int32, ctypes.c_int32] + [ptr] * 5 + [
                ctypes.c_int64,
                ctypes.c_int32,
                ctypes.c_int32,
                ctypes.c_int32,
            ]
            last = getattr(lib, "lstm2_oracle_last_output_" + suffix)
            last.restype = ctypes.c_int
            last.argtypes = [ptr] * 3 + [ctypes.c_int32, ctypes.c_int32, ptr, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
            bwd = getattr(lib, "lstm2_oracle_bwd_" + suffix)
            bwd.restype = ctypes.c_int
            bwd.argtypes = [ptr] * 5 + [ctypes.c_int32, ctypes.c_int32] + [ptr] * 9 + [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
            gb = getattr(lib, "lstm_generic_base_oracle_fwd_" + suffix)
            gb.restype = ctypes.c_int
            gb.argtypes = [ptr] * 7 + [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
            gbb = getattr(lib, "lstm_generic_base_oracle_bwd_" + suffix)
            gbb.restype = ctypes.c_int
            gbb.argtypes = [ptr] * 10 + [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
            lm = getattr(lib, "lstm_low_mem_oracle_fwd_" + suffix)
            lm.restype = ctypes.c_int
            lm.argtypes = [ptr] * 6 + [ctypes.c_int32, ctypes.c_int32] + [ptr] * 3 + [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32]
        lib.lstm2_oracle_max_threads.restype = ctypes.c_int
        fp = ctypes.POINTER(ctypes.c_float)
        lib.lstm2_oracle_pointwise_f32.restype = None
        lib.lstm2_oracle_pointwise_f32.argtypes = [ctypes.c_int32, ctypes.c_int32] + [fp] * 7
        lib.lstm2_oracle_bwd_pointwise_f32.restype = None
        lib.lstm2_oracle_bwd_pointwise_f32.argtypes = [ctypes.c_int32, ctypes.c_int32] + [fp] * 8
        _lib = lib
    return _lib


def max_threads() -> int:
    """Number of OpenMP threads the GEMM part can use on this host."""
    return int(_load().lstm2_oracle_max_threads())


def _prep(a, dtype, shape, name):
    a = numpy.ascontiguousarray(a, dtype=dtype)
    if a.shape != shape:
        raise ValueError("oracle: %s has shape %r, expected %r" % (name, a.shape, shape))
    return a


def native_lstm2_fwd(
    X, W, y0, c0, i, start: int = 0, step: int = 1, *, dtype=numpy.float32, threads: int = 1
) -> Tuple[numpy.ndarray, numpy.ndarray, numpy.ndarray, numpy.ndarray, numpy.ndarray]:
    """
    Reference semantics of ``NativeLstm2`` forward (returnn/native_op.py:1184-1285).

    :param X: [T,B,4n] pre-projected gate inputs, gate order cell-in, input, forget, output
    :param W: [n,4n] recurrent weights
    :param y0: [B,n] initial output
    :param c0: [B,n] initial cell state
    :param i: [T,B] 0/1 mask
    :param start: first frame (for step<0 counted from the end)
    :param step: +-1 direction, or a wider stride
    :param dtype: numpy.float32 (the reference's arithmetic) or numpy.float64
    :param threads: OpenMP threads for the recurrent GEMM; the pointwise part is always sequential
    :return: Y [T,B,n], C [T,B,n], H [T,B,4n], d [B,n], y_last [B,n]
      (y_last is the final carry of the last valid output, not an output of the reference op:
      it is what the caller derives with ``_lstm_last_output``, returnn/tf/native_op.py:913-929)
    """
    dtype = numpy.dtype(dtype)
    if dtype == numpy.float32:
        suffix, ctype = "f32", ctypes.c_float
    elif dtype == numpy.float64:
        suffix, ctype = "f64", ctypes.c_double
    else:
        raise ValueError("oracle: dtype must be float32 or float64")
    i = numpy.ascontiguousarray(i, dtype=dtype)
    y0 = numpy.ascontiguousarray(y0, dtype=dtype)
    if i.ndim != 2 or y0.ndim != 2:
        raise ValueError("oracle: i must be [T,B] and y0 [B,n]")
    T, B = i.shape
    n = y0.shape[1]
    X = _prep(X, dtype, (T, B, 4 * n), "X")
    W = _prep(W, dtype, (n, 4 * n), "W")
    y0 = _prep(y0, dtype, (B, n), "y0")
    c0 = _prep(c0, dtype, (B, n), "c0")
    Y = numpy.empty((T, B, n), dtype=dtype)
    C = numpy.empty((T, B, n), dtype=dtype)
    H = numpy.empty((T, B, 4 * n), dtype=dtype)
    d = numpy.empty((B, n), dtype=dtype)
    y_last = numpy.empty((B, n), dtype=dtype)
    p = ctypes.POINTER(ctype)
    fwd = getattr(_load(), "lstm2_oracle_fwd_" + suffix)
    rc = fwd(
        *(a.ctypes.data_as(p) for a in (X, W, y0, c0, i)),
        int(start),
        int(step),
        *(a.ctypes.data_as(p) for a in (Y, C, H, d, y_last)),
        T,
        B,
        n,
        int(threads),
    )
    if rc == 2:
        raise ValueError("oracle: need 0 <= start < T and step != 0 (start=%r, step=%r, T=%r)" % (start, step, T))
    if rc != 0:
        raise RuntimeError("oracle: error code %i" % rc)
    return Y, C, H, d, y_last


def lstm_last_output(Y, y0, i, start: int = 0, step: int = 1, *, dtype=numpy.float32) -> numpy.ndarray:
    """
    Caller-side final output per sequence (returnn/tf/native_op.py:913-929).

    :param Y: [T,B,n] op output
    :param y0: [B,n]
    :param i: [T,B] mask
    :return: [B,n]
    """
    dtype = numpy.dtype(dtype)
    suffix, ctype = ("f32", ctypes.c_float) if dtype == numpy.float32 else ("f64", ctypes.c_double)
    Y = numpy.ascontiguousarray(Y, dtype=dtype)
    T, B, n = Y.shape
    y0 = _prep(y0, dtype, (B, n), "y0")
    i = _prep(i, dtype, (T, B), "i")
    out = numpy.empty((B, n), dtype=dtype)
    p = ctypes.POINTER(ctype)
    rc = getattr(_load(), "lstm2_oracle_last_output_" + suffix)(
        Y.ctypes.data_as(p), y0.ctypes.data_as(p), i.ctypes.data_as(p), int(start), int(step), out.ctypes.data_as(p), T, B, n
    )
    if rc != 0:
        raise ValueError("oracle: last_output error code %i" % rc)
    return out


def native_lstm2_fwd_blas(X, W, y0, c0, i, start: int = 0, step: int = 1):
    """
    Same op, float32, with the structure of the reference's CPU path: per visited frame one SGEMM
    ``H[t] += y_prev . W`` through the BLAS numpy links (multi-threaded, like the reference's GEMM back-ends,
    returnn/native_op.cpp:535-620) followed by the sequential pointwise kernel of ``oracle/lstm2_oracle.c``.
    This is the variant the benchmark times as the CPU baseline; it agrees with :func:`native_lstm2_fwd`
    up to the summation order inside the BLAS.

    :return: Y, C, H, d, y_last as in :func:`native_lstm2_fwd`
    """
    f32 = numpy.float32
    i = numpy.ascontiguousarray(i, dtype=f32)
    y0 = numpy.ascontiguousarray(y0, dtype=f32)
    T, B = i.shape
    n = y0.shape[1]
    X = _prep(X, f32, (T, B, 4 * n), "X")
    W = _prep(W, f32, (n, 4 * n), "W")
    c0 = _prep(c0, f32, (B, n), "c0")
    Y = numpy.zeros((T, B, n), dtype=f32)
    C = numpy.zeros((T, B, n), dtype=f32)
    d = numpy.zeros((B, n), dtype=f32)
    if T == 0:
        return Y, C, numpy.zeros((T, B, 4 * n), dtype=f32), c0.copy(), y0.copy()
    if not (0 <= start < T) or step == 0:
        raise ValueError("oracle: need 0 <= start < T and step != 0 (start=%r, step=%r, T=%r)" % (start, step, T))
    H = X.copy()
    y_prev = numpy.empty((B, n), dtype=f32)
    first, end = (start, T - 1) if step > 0 else (T - start - 1, 0)
    pointwise = _load().lstm2_oracle_pointwise_f32
    fp = ctypes.POINTER(ctypes.c_float)
    ptr = lambda a: a.ctypes.data_as(fp)  # noqa: E731
    t = first
    while (t <= end) if step > 0 else (t >= end):
        y_in = y0 if t == first else y_prev
        c_in = c0 if t == first else C[t - step]
        H[t] += y_in @ W
        pointwise(B, n, ptr(i[t]), ptr(H[t]), ptr(y_in), ptr(c_in), ptr(Y[t]), ptr(C[t]), ptr(y_prev))
        t += step
    d[...] = C[t - step]
    return Y, C, H, d, y_prev


def native_lstm2_bwd(X, W, y0, c0, i, start, step, Y, C, H, DY, Dd, *, dtype=numpy.float32):
    """
    Reference semantics of the ``NativeLstm2`` gradient op (returnn/native_op.py:1288-1464, inputs as
    ``grad_input_map`` :1071-1077 arranges them).

    :param X, W, y0, c0, i, start, step: the forward op's inputs
    :param Y, C, H: the forward op's outputs (H = activated gates)
    :param DY: [T,B,n] error signal on Y
    :param Dd: [B,n] error signal on the final cell state
    :return: DX [T,B,4n], DW [n,4n], Dy0 [B,n], Dc0 [B,n]
    """
    dtype = numpy.dtype(dtype)
    if dtype == numpy.float32:
        suffix, ctype = "f32", ctypes.c_float
    elif dtype == numpy.float64:
        suffix, ctype = "f64", ctypes.c_double
    else:
        raise ValueError("oracle: dtype must be float32 or float64")
    i = numpy.ascontiguousarray(i, dtype=dtype)
    y0 = numpy.ascontiguousarray(y0, dtype=dtype)
    T, B = i.shape
    n = y0.shape[1]
    X = _prep(X, dtype, (T, B, 4 * n), "X")
    W = _prep(W, dtype, (n, 4 * n), "W")
    c0 = _prep(c0, dtype, (B, n), "c0")
    Y = _prep(Y, dtype, (T, B, n), "Y")
    C = _prep(C, dtype, (T, B, n), "C")
    H = _prep(H, dtype, (T, B, 4 * n), "H")
    DY = _prep(DY, dtype, (T, B, n), "DY")
    Dd = _prep(Dd, dtype, (B, n), "Dd")
    DX = numpy.zeros((T, B, 4 * n), dtype=dtype)
    DW = numpy.empty((n, 4 * n), dtype=dtype)
    Dy0 = numpy.empty((B, n), dtype=dtype)
    Dc0 = numpy.empty((B, n), dtype=dtype)
    p = ctypes.POINTER(ctype)
    bwd = getattr(_load(), "lstm2_oracle_bwd_" + suffix)
    rc = bwd(
        *(a.ctypes.data_as(p) for a in (X, W, y0, c0, i)), int(start), int(step),
        *(a.ctypes.data_as(p) for a in (Y, C, H, DY, Dd, DX, DW, Dy0, Dc0)), T, B, n,
    )  # fmt: skip
    if rc == 2:
        raise ValueError("oracle: need 0 <= start < T and step != 0 (start=%r, step=%r, T=%r)" % (start, step, T))
    if rc != 0:
        raise RuntimeError("oracle: error code %i" % rc)
    return DX, DW, Dy0, Dc0


def native_lstm2_bwd_blas(W, y0, c0, i, start, step, Y, C, H, DY, Dd):
    """
    The gradient op in float32 with the structure of the reference's CPU path: per visited frame the sequential
    pointwise kernel, then ``Dy0 += DX[t] . W^T`` through the BLAS numpy links; afterwards the weight gradient as one
    large GEMM (``|step| == 1``) or one per frame, and ``y0^T . dx0`` (returnn/native_op.py:1365-1462).  This is the
    variant the benchmark times as the CPU baseline of the gradient op; it agrees with :func:`native_lstm2_bwd` up to
    the summation order inside the BLAS.
    """
    f32 = numpy.float32
    i = numpy.ascontiguousarray(i, dtype=f32)
    y0 = numpy.ascontiguousarray(y0, dtype=f32)
    T, B = i.shape
    n = y0.shape[1]
    W = _prep(W, f32, (n, 4 * n), "W")
    c0 = _prep(c0, f32, (B, n), "c0")
    Y = _prep(Y, f32, (T, B, n), "Y")
    C = _prep(C, f32, (T, B, n), "C")
    H = _prep(H, f32, (T, B, 4 * n), "H")
    DY = _prep(DY, f32, (T, B, n), "DY")
    DX = numpy.zeros((T, B, 4 * n), dtype=f32)
    DW = numpy.zeros((n, 4 * n), dtype=f32)
    Dy0 = numpy.zeros((B, n), dtype=f32)
    Dc0 = _prep(Dd, f32, (B, n), "Dd").copy()
    if T == 0:
        return DX, DW, Dy0, Dc0
    if not (0 <= start < T) or step == 0:
        raise ValueError("oracle: need 0 <= start < T and step != 0 (start=%r, step=%r, T=%r)" % (start, step, T))
    dx0 = numpy.zeros((B, 4 * n), dtype=f32)
    abs_step = abs(step)
    num_steps = (T - start + abs_step - 1) // abs_step
    first = start if step > 0 else T - start - 1
    end = first + (num_steps - 1) * step
    pointwise = _load().lstm2_oracle_bwd_pointwise_f32
    fp = ctypes.POINTER(ctypes.c_float)
    ptr = lambda a: a.ctypes.data_as(fp)  # noqa: E731
    WT = numpy.ascontiguousarray(W.T)
    for t in range(end, first - step, -step):
        prev_c = C[t - step] if t != first else c0
        pointwise(B, n, ptr(i[t]), ptr(H[t]), ptr(prev_c), ptr(DY[t]), ptr(Dy0), ptr(Dc0), ptr(DX[t]), ptr(dx0))
        Dy0 += DX[t] @ WT
    if num_steps > 1:
        if abs_step == 1:
            lo = min(first, end)
            ys = Y[lo + max(0, -step) : lo + max(0, -step) + num_steps - 1].reshape(-1, n)
            dxs = DX[lo + max(0, step) : lo + max(0, step) + num_steps - 1].reshape(-1, 4 * n)
            DW += ys.T @ dxs
        else:
            for t in range(end - step, first - step, -step):
                DW += Y[t].T @ DX[t + step]
    DW += y0.T @ dx0
    return DX, DW, Dy0, Dc0


def _suffix(dtype):
    dtype = numpy.dtype(dtype)
    if dtype == numpy.float32:
        return dtype, "f32", ctypes.c_float
    if dtype == numpy.float64:
        return dtype, "f64", ctypes.c_double
    raise ValueError("oracle: dtype must be float32 or float64")


def lstm_generic_base_fwd(Z, V_h, c, i, *, dtype=numpy.float32):
    """
    Reference semantics of ``LstmGenericBase`` forward (returnn/native_op.py:381-429, :486-523).

    :param Z: [T,B,4n] gate inputs (cell-in, input, forget, output)
    :param V_h: [n,4n]
    :param c: [B,n] initial cell state
    :param i: [T,B] 0/1 mask
    :return: Y [T,B,n], H [T,B,4n] (cell state, then the activated input, forget, output gates), d [B,n]
    """
    dtype, suffix, ctype = _suffix(dtype)
    i = numpy.ascontiguousarray(i, dtype=dtype)
    c = numpy.ascontiguousarray(c, dtype=dtype)
    T, B = i.shape
    n = c.shape[1]
    Z = _prep(Z, dtype, (T, B, 4 * n), "Z")
    V_h = _prep(V_h, dtype, (n, 4 * n), "V_h")
    Y = numpy.zeros((T, B, n), dtype=dtype)
    H = numpy.zeros((T, B, 4 * n), dtype=dtype)
    d = numpy.zeros((B, n), dtype=dtype)
    p = ctypes.POINTER(ctype)
    rc = getattr(_load(), "lstm_generic_base_oracle_fwd_" + suffix)(*(a.ctypes.data_as(p) for a in (Z, V_h, c, i, Y, H, d)), T, B, n)
    if rc != 0:
        raise ValueError("oracle: LstmGenericBase needs T > 0")
    return Y, H, d


def lstm_generic_base_bwd(V_h, c, i, Y, H, DY, Dd, *, dtype=numpy.float32):
    """
    Reference semantics of the ``LstmGenericBase`` gradient op (returnn/native_op.py:430-485, :525-574; inputs as its
    ``grad_input_map`` :374-378).

    :param Y, H: results of the forward pass
    :param DY: [T,B,n] error signal on Y; Dd: [B,n] error signal on the final cell state
    :return: DZ [T,B,4n], DV_h [n,4n], Dc [B,n]
    """
    dtype, suffix, ctype = _suffix(dtype)
    i = numpy.ascontiguousarray(i, dtype=dtype)
    c = numpy.ascontiguousarray(c, dtype=dtype)
    T, B = i.shape
    n = c.shape[1]
    V_h = _prep(V_h, dtype, (n, 4 * n), "V_h")
    Y = _prep(Y, dtype, (T, B, n), "Y")
    H = _prep(H, dtype, (T, B, 4 * n), "H")
    DY = _prep(DY, dtype, (T, B, n), "DY")
    Dd = _prep(Dd, dtype, (B, n), "Dd")
    DZ = numpy.zeros((T, B, 4 * n), dtype=dtype)
    DV_h = numpy.zeros((n, 4 * n), dtype=dtype)
    Dc = numpy.zeros((B, n), dtype=dtype)
    p = ctypes.POINTER(ctype)
    rc = getattr(_load(), "lstm_generic_base_oracle_bwd_" + suffix)(
        *(a.ctypes.data_as(p) for a in (V_h, c, i, Y, H, DY, Dd, DZ, DV_h, Dc)), T, B, n
    )
    if rc != 0:
        raise ValueError("oracle: LstmGenericBase gradient needs T > 0")
    return DZ, DV_h, Dc


def lstm_low_mem_fwd(X, W, b, y0, c0, i, start: int = 0, step: int = 1, *, dtype=numpy.float32):
    """
    Reference semantics of ``LstmLowMem`` forward (returnn/native_op.py:624-655, :771-836).

    :param X: [T,B,n_in]
    :param W: [n_in+n,4n] input weights stacked on recurrent weights
    :param b: [4n]
    :return: Y [T,B,n], C [T,B,n], d [B,n]
    """
    dtype, suffix, ctype = _suffix(dtype)
    i = numpy.ascontiguousarray(i, dtype=dtype)
    y0 = numpy.ascontiguousarray(y0, dtype=dtype)
    T, B = i.shape
    n = y0.shape[1]
    X = numpy.ascontiguousarray(X, dtype=dtype)
    n_in = X.shape[2]
    X = _prep(X, dtype, (T, B, n_in), "X")
    W = _prep(W, dtype, (n_in + n, 4 * n), "W")
    b = _prep(b, dtype, (4 * n,), "b")
    c0 = _prep(c0, dtype, (B, n), "c0")
    Y = numpy.zeros((T, B, n), dtype=dtype)
    C = numpy.zeros((T, B, n), dtype=dtype)
    d = numpy.zeros((B, n), dtype=dtype)
    p = ctypes.POINTER(ctype)
    rc = getattr(_load(), "lstm_low_mem_oracle_fwd_" + suffix)(
        *(a.ctypes.data_as(p) for a in (X, W, b, y0, c0, i)), int(start), int(step), *(a.ctypes.data_as(p) for a in (Y, C, d)), T, B, n_in, n
    )
    if rc == 2:
        raise ValueError("oracle: need 0 <= start < T and step != 0 (start=%r, step=%r, T=%r)" % (start, step, T))
    if rc == 4:
        raise ValueError("oracle: LstmLowMem with step < 0 runs from frame T-start-1 down to frame start; start=%r visits nothing" % start)
    if rc != 0:
        raise RuntimeError("oracle: error code %i" % rc)
    return Y, C, d


def lstm_low_mem_bwd(X, W, b, y0, c0, i, start, step, Y, C, DY, Dd, *, dtype=numpy.float64):
    """
    Reference semantics of the ``LstmLowMem`` gradient op: the host loop of returnn/native_op.py:958-1020 with its
    pointwise kernel :659-712, restated in numpy frame by frame (inputs as ``grad_input_map`` :619-625).  The gates are
    recomputed from X, Y, W and b; the forward pass stores only Y and C.

    Pinned for masks without holes before the last valid frame in processing order (full-length batches in both
    directions, right-padded batches with step > 0) by finite differences of the pinned forward oracle and by torch
    autograd (tests/test_oracle_siblings.py).  On a masked frame with valid frames behind it in the recurrence the
    reference's kernel lets the error of the output through unmasked (``d_y_b = d_y * mask + d_h``, :679; its own
    comment :965 calls the mask handling unfinished): what this function returns there is the literal restatement and
    nothing else pins it -- parity unpinned for such masks.

    The reference's loop starts at frame T-1 (step > 0) or at frame ``start`` (step < 0) whatever the stride; that is
    the frame set of the forward pass only if the stride divides the distance between the two ends.  Other cases are
    refused here (ValueError), as in the HIP entry.

    :return: DX [T,B,n_in], DW [n_in+n,4n], Db [4n], Dh [B,n] (error of y0), Dc [B,n] (error of c0)
    """
    dtype = numpy.dtype(dtype).type
    i = numpy.ascontiguousarray(i, dtype=dtype)
    T, B = i.shape
    y0 = numpy.ascontiguousarray(y0, dtype=dtype)
    n = y0.shape[1]
    X = numpy.ascontiguousarray(X, dtype=dtype)
    n_in = X.shape[2]
    W = _prep(W, dtype, (n_in + n, 4 * n), "W")
    b = _prep(b, dtype, (4 * n,), "b")
    c0 = _prep(c0, dtype, (B, n), "c0")
    Y = _prep(Y, dtype, (T, B, n), "Y")
    C = _prep(C, dtype, (T, B, n), "C")
    DY = _prep(DY, dtype, (T, B, n), "DY")
    Dd = _prep(Dd, dtype, (B, n), "Dd")
    if not (T > 0 and 0 <= start < T and step != 0):
        raise ValueError("oracle: need T > 0, 0 <= start < T and step != 0 (start=%r, step=%r, T=%r)" % (start, step, T))
    DX = numpy.zeros((T, B, n_in), dtype=dtype)
    DW = numpy.zeros((n_in + n, 4 * n), dtype=dtype)
    Db = numpy.zeros((4 * n,), dtype=dtype)
    Dh = numpy.zeros((B, n), dtype=dtype)
    Dc = Dd.copy()
    end = T - 1
    if step < 0:
        end = start
        start = T - start - 1
    if (step > 0 and (end - start) % step != 0) or (step < 0 and (start < end or (start - end) % (-step) != 0)):
        raise ValueError("oracle: LstmLowMem gradient: the stride does not divide the distance between the first and the last frame")
    one = dtype(1)

    def sigmoid(z):
        return one / (one + numpy.exp(-z))

    t = end
    while (t >= start) if step > 0 else (t <= start):
        right = (t - step >= start) if step > 0 else (t - step <= start)
        x_h = numpy.concatenate([X[t], Y[t - step] if right else y0], axis=1)
        intern = x_h @ W + b[None, :]
        prev_c = C[t - step] if right else c0
        m = i[t][:, None]
        d_y_b = DY[t] * m + Dh
        d_c_b = Dc * m
        cell_in, inp, fgt, out = numpy.tanh(intern[:, :n]), sigmoid(intern[:, n : 2 * n]), sigmoid(intern[:, 2 * n : 3 * n]), sigmoid(intern[:, 3 * n :])
        gc = numpy.tanh(prev_c * fgt + cell_in * inp)
        d_out = (one - out) * out * gc * d_y_b
        d_c2 = d_c_b + out * d_y_b * (one - gc * gc)
        d_cell_in = (one - cell_in * cell_in) * inp * d_c2
        d_inp = (one - inp) * inp * cell_in * d_c2
        d_fgt = (one - fgt) * fgt * prev_c * d_c2
        Dc = fgt * d_c2 + Dc * (one - m)
        d_intern = numpy.concatenate([d_cell_in, d_inp, d_fgt, d_out], axis=1)
        Db += d_intern.sum(axis=0)
        dx_h = d_intern @ W.T
        DW += x_h.T @ d_intern
        DX[t] = dx_h[:, :n_in]
        Dh = dx_h[:, n_in:]
        t -= step
    return DX, DW, Db, Dh, Dc
