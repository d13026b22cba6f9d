"""
Ops compiled by the HIP op loader from source in the native-op dialect, run on the GPU through their C entry points and
checked against numpy restatements.  The ops are tests/dialect_ops.py; their shared objects are built on the CPU
beforehand (tests/test_op_loader.py or the build entry point) and found again by content hash.

float32 throughout: rtol 1e-5 / atol 1e-6 where sums are short, 1e-4 relative for the GEMM results (rocBLAS summation
order differs from numpy's); integer outputs exact.
"""

from __future__ import annotations

import ctypes

import numpy
import pytest
import torch
from numpy.testing import assert_allclose, assert_array_equal

import dialect_ops
from returnn_amd import op_loader, torch_native_op
from _gpu_util import announce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a, dtype=numpy.float32):
    return torch.from_numpy(numpy.ascontiguousarray(a, dtype=dtype)).to(DEV)


def host(*tensors):
    torch.cuda.synchronize()
    return tuple(t.cpu().numpy() for t in tensors)


def elman_numpy(X, W, h0, mask, start, step):
    T = X.shape[0]
    Y = numpy.zeros_like(X, dtype=numpy.float64)
    h = h0.astype(numpy.float64)
    t = start if step > 0 else T - 1 - start
    while 0 <= t < T:
        m = mask[t][:, None]
        h = m * numpy.tanh(X[t] + h @ W) + (1 - m) * h
        Y[t] = h
        t += step
    return Y, h


@pytest.mark.parametrize("start,step", [(0, 1), (0, -1), (1, 2), (2, -3)])
def test_elman_scan(start, step):
    announce("op_loader elman_scan", start, step)
    rng = numpy.random.default_rng(7)
    T, B, n = 13, 5, 48
    X = rng.normal(0, 0.5, (T, B, n)).astype(numpy.float32)
    W = (rng.uniform(-1, 1, (n, n)) / numpy.sqrt(n)).astype(numpy.float32)
    h0 = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    mask = (rng.random((T, B)) < 0.7).astype(numpy.float32)
    op = torch_native_op.make_op(dialect_ops.ElmanScan)
    assert op is torch.ops.ElmanScan.ElmanScan
    Y, hT = host(*op(dev(X), dev(W), dev(h0), dev(mask), start, step))
    Y2, h2 = elman_numpy(X, W, h0, mask, start, step)
    assert_allclose(Y, Y2, rtol=1e-4, atol=1e-5)
    assert_allclose(hT, h2, rtol=1e-4, atol=1e-5)


def test_elman_scan_failed_check_is_an_exception():
    """A failed assert_cmp in the op code raises, names the values, releases the op's temporaries; the next call works."""
    announce("op_loader elman_scan failed check")
    op = torch_native_op.make_op(dialect_ops.ElmanScan)
    X, W, h0, mask = torch.zeros(3, 2, 8, device=DEV), torch.zeros(8, 8, device=DEV), torch.zeros(2, 8, device=DEV), torch.ones(3, 2, device=DEV)
    with pytest.raises(RuntimeError, match=r"Ndarray_DIMS\(W\)\[0\] == width, 4 == 8"):
        op(X, torch.zeros(4, 8, device=DEV), h0, mask, 0, 1)
    with pytest.raises(RuntimeError, match=r"first < frames, 3 < 3"):
        op(X, W, h0, mask, 3, 1)
    with pytest.raises(RuntimeError, match="shape ndim is not 3"):
        op(X[0], W, h0, mask, 0, 1)
    Y, hT = host(*op(X, W, h0, mask, 0, 1))
    assert numpy.abs(Y).max() == 0 and numpy.abs(hT).max() == 0


def test_row_log_sum_exp():
    announce("op_loader row_log_sum_exp")
    rng = numpy.random.default_rng(3)
    op = torch_native_op.make_op(dialect_ops.RowLogSumExp)
    for rows, cols in [(1, 1), (7, 5), (33, 1000), (4, 257)]:
        x = rng.normal(0, 3, (rows, cols)).astype(numpy.float32)
        lse, arg = op(dev(x))
        assert arg.dtype == torch.int32 and lse.dtype == torch.float32
        lse, arg = host(lse, arg)
        x64 = x.astype(numpy.float64)
        want = numpy.log(numpy.exp(x64 - x64.max(1, keepdims=True)).sum(1)) + x64.max(1)
        assert_allclose(lse, want, rtol=1e-5, atol=1e-6)
        assert_array_equal(arg, x.argmax(1))
    with pytest.raises(RuntimeError, match="the op code gave up"):
        op(torch.zeros(3, 0, device=DEV))
    # converted and made contiguous on the way in (float64, transposed view)
    xt = torch.from_numpy(rng.normal(0, 1, (6, 9))).to(DEV).t()
    lse, arg = host(*op(xt))
    x64 = xt.cpu().numpy()
    assert_allclose(lse, numpy.log(numpy.exp(x64).sum(1)), rtol=1e-5)


def test_bucket_sum_in_place_and_dummy_out():
    announce("op_loader bucket_sum")
    rng = numpy.random.default_rng(5)
    N, K = 5000, 37
    values = rng.normal(0, 1, N).astype(numpy.float32)
    idx = rng.integers(-2, K + 2, N)  # some out of range: skipped
    acc0 = rng.normal(0, 1, K).astype(numpy.float32)
    op = torch_native_op.make_op(dialect_ops.BucketSum)
    acc, vals = dev(acc0), dev(values)
    out, hits, doubled = op(acc, vals, dev(idx, numpy.int64))  # int64 indices are converted to the declared int32
    assert out.data_ptr() == acc.data_ptr() and doubled.data_ptr() == vals.data_ptr()  # worked in place
    out, hits, doubled = host(out, hits, doubled)
    ok = (idx >= 0) & (idx < K)
    want = acc0.astype(numpy.float64)
    numpy.add.at(want, idx[ok], values[ok].astype(numpy.float64))
    assert_allclose(out, want, rtol=1e-4, atol=1e-4)
    assert_array_equal(hits, numpy.bincount(idx[ok], minlength=K).astype(numpy.float32))
    assert_array_equal(doubled, values * 2)
    with pytest.raises(RuntimeError, match="BucketSum: 5000 values but 3 indices"):
        op(dev(acc0), dev(values), dev(idx[:3], numpy.int32))


def test_affine_helpers():
    announce("op_loader affine_all")
    rng = numpy.random.default_rng(9)
    T, B, n, m = 6, 4, 10, 7
    A = rng.normal(0, 1, (T, B, n)).astype(numpy.float32)
    Bm = rng.normal(0, 1, (T, B, m)).astype(numpy.float32)
    V = rng.normal(0, 1, (n, m)).astype(numpy.float32)
    op = torch_native_op.make_op(dialect_ops.AffineAll)
    AtB, AtB_shift, AV, VtV = host(*op(dev(A), dev(Bm), dev(V)))
    A64, B64, V64 = A.astype(numpy.float64), Bm.astype(numpy.float64), V.astype(numpy.float64)
    assert_allclose(AtB, numpy.einsum("tbn,tbm->nm", A64, B64), rtol=1e-4, atol=1e-4)
    assert_allclose(AtB_shift, numpy.einsum("tbn,tbm->nm", A64[:-1], B64[1:]), rtol=1e-4, atol=1e-4)
    assert_allclose(AV, A64 @ V64, rtol=1e-4, atol=1e-4)
    assert_allclose(VtV, V64.T @ V64, rtol=1e-4, atol=1e-4)


def test_fake_impl_and_schema():
    announce("op_loader schema")
    torch_native_op.make_op(dialect_ops.BucketSum)
    schema = str(torch.ops.BucketSum.BucketSum.default._schema)
    assert "Tensor acc, Tensor values, Tensor idx" in schema and schema.count("Tensor") == 6  # the dummy output is returned too
    torch_native_op.make_op(dialect_ops.ElmanScan)
    assert "int start, int step" in str(torch.ops.ElmanScan.ElmanScan.default._schema)
    from torch._subclasses.fake_tensor import FakeTensorMode

    op = torch_native_op.make_op(dialect_ops.RowLogSumExp)
    with FakeTensorMode():
        lse, arg = op(torch.empty(5, 11, device=DEV))
        assert tuple(lse.shape) == (5,) and arg.dtype == torch.int32


def test_c_abi_with_the_library_allocator():
    """Direct call of the C entry point with no allocator callbacks: device_malloc falls back to hipMallocAsync on the stream."""
    announce("op_loader c_abi hipMallocAsync")
    rng = numpy.random.default_rng(11)
    T, B, n = 4, 3, 16
    X = rng.normal(0, 0.5, (T, B, n)).astype(numpy.float32)
    W = (rng.uniform(-1, 1, (n, n)) / 4).astype(numpy.float32)
    h0 = numpy.zeros((B, n), numpy.float32)
    mask = numpy.ones((T, B), numpy.float32)
    op = op_loader.compile_op(dialect_ops.ElmanScan)
    lib = op.lib()
    tensors = [dev(X), dev(W), dev(h0), dev(mask)]
    Y, hT = torch.zeros(T, B, n, device=DEV), torch.zeros(B, n, device=DEV)
    keep = []

    def rec(t=None, scalar=None):
        r = op_loader.RtnNdarray()
        if t is None:
            cell = ctypes.c_int32(scalar)
            keep.append(cell)
            r.data, r.ndim, r.elem_size, r.on_host = ctypes.cast(ctypes.pointer(cell), ctypes.c_void_p), 0, 4, 1
        else:
            dims = (ctypes.c_int64 * t.dim())(*t.shape)
            keep.append(dims)
            r.data, r.dims, r.ndim, r.elem_size = t.data_ptr(), dims, t.dim(), 4
        return r

    ins = (op_loader.RtnNdarray * 6)(*[rec(t) for t in tensors], rec(scalar=0), rec(scalar=1))
    outs = (op_loader.RtnNdarray * 2)(rec(Y), rec(hT))
    host_rec = op_loader.RtnOpHost()
    host_rec.stream = torch.cuda.current_stream().cuda_stream
    rc = lib.ElmanScan_fw(ctypes.byref(host_rec), 6, ins, 2, outs)
    assert rc == 0, lib.ElmanScan_last_error()
    Yh, hTh = host(Y, hT)
    Y2, h2 = elman_numpy(X, W, h0, mask, 0, 1)
    assert_allclose(Yh, Y2, rtol=1e-4, atol=1e-5)
    assert_allclose(hTh, h2, rtol=1e-4, atol=1e-5)


def elman_torch(X, W, h0, mask, start, step):
    """The scan in differentiable torch float64 (CPU): autograd through it is the independent check of c_bw_code."""
    T = X.shape[0]
    ys = [torch.zeros_like(X[0]) for _ in range(T)]
    h = h0
    t = start if step > 0 else T - 1 - start
    while 0 <= t < T:
        m = mask[t][:, None]
        h = m * torch.tanh(X[t] + h @ W) + (1 - m) * h
        ys[t] = h
        t += step
    return torch.stack(ys), h


@pytest.mark.parametrize("start,step", [(0, 1), (0, -1), (1, 2)])
def test_gradient_op_through_autograd(start, step):
    """make_op_with_grad: forward op + derived gradient op under torch.autograd, against autograd through plain torch."""
    announce("op_loader gradient", start, step)
    rng = numpy.random.default_rng(21)
    T, B, n = 9, 4, 24
    X = rng.normal(0, 0.5, (T, B, n))
    W = rng.uniform(-1, 1, (n, n)) / numpy.sqrt(n)
    h0 = rng.normal(0, 0.3, (B, n))
    mask = (rng.random((T, B)) < 0.7).astype(numpy.float64)
    R1, R2 = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    ref = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (X, W, h0)]
    Yr, hr = elman_torch(ref[0], ref[1], ref[2], torch.tensor(mask), start, step)
    ((Yr * torch.tensor(R1)).sum() + (hr * torch.tensor(R2)).sum()).backward()

    op = torch_native_op.make_op_with_grad(dialect_ops.ElmanScan)
    got = [dev(a).requires_grad_(True) for a in (X, W, h0)]
    Y, hT = op(got[0], got[1], got[2], dev(mask), start, step)
    ((Y * dev(R1)).sum() + (hT * dev(R2)).sum()).backward()
    torch.cuda.synchronize()
    assert_allclose(Y.detach().cpu().numpy(), Yr.detach().numpy(), rtol=1e-4, atol=1e-5)
    for name, g, r in zip(("DX", "DW", "Dh0"), got, ref):
        scale = float(r.grad.abs().max())
        assert_allclose(g.grad.cpu().numpy(), r.grad.numpy(), rtol=0, atol=2e-5 * max(scale, 1.0), err_msg=name)
    # an output nobody differentiates gets a zero gradient: only hT contributes
    got2 = [dev(a).requires_grad_(True) for a in (X, W, h0)]
    _, hT2 = op(got2[0], got2[1], got2[2], dev(mask), start, step)
    (hT2 * dev(R2)).sum().backward()
    ref2 = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (X, W, h0)]
    (elman_torch(ref2[0], ref2[1], ref2[2], torch.tensor(mask), start, step)[1] * torch.tensor(R2)).sum().backward()
    torch.cuda.synchronize()
    assert_allclose(got2[1].grad.cpu().numpy(), ref2[1].grad.numpy(), rtol=0, atol=2e-5 * max(float(ref2[1].grad.abs().max()), 1.0))
