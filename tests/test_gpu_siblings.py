"""
Parity of the sibling ops' forward pass on the GPU (LstmGenericBase, LstmLowMem; returnn/native_op.py:333-523, :577-836)
with their CPU oracle, through the C ABI.

Both run on the NativeLstm2 kernels with two switches: the recurrent input of a frame is the masked output of the frame
before (no carry over masked frames), and LstmGenericBase keeps the cell state where NativeLstm2 keeps the activated
cell input.  The masks here have holes in the middle of sequences, the only place where the switches show.

Tolerances as for NativeLstm2: float32 ``rtol=1e-5, atol=2e-6``; bfloat16 ``atol=2e-2`` against the float32 oracle on the
same float32 inputs (LstmLowMem's input projection adds two roundings to bfloat16, which is why its inputs are kept
small enough for that bound to hold).
"""

from __future__ import annotations

import numpy
import pytest
import torch
from numpy.testing import assert_allclose

from oracle import lstm2_oracle as oracle
from returnn_amd import lib, native_op, torch_native_op
from _gpu_util import announce, get_op, to_dev
from _textbook import visited_slice

pytestmark = pytest.mark.gpu

F32_RTOL, F32_ATOL = 1e-5, 2e-6
BF16_ATOL = 2e-2


def _check(got, want, dtype, what):
    for name, g, w in zip(what[1], got, want):
        assert g.shape == w.shape, (what, name)
        assert numpy.all(numpy.isfinite(g)), (what, name)
        if dtype == "f32":
            assert_allclose(g, w, rtol=F32_RTOL, atol=F32_ATOL, err_msg="%s %s" % (what[0], name))
        else:
            assert_allclose(g, w, rtol=0, atol=BF16_ATOL, err_msg="%s %s" % (what[0], name))


def _holes(rng, T, B, p_keep=0.7):
    return (rng.random((T, B)) < p_keep).astype(numpy.float32)


def run_generic_base(Z, V_h, c, i, *, dtype="f32", mode="auto"):
    get_op()  # builds the library if needed
    op = torch_native_op.make_op(native_op.LstmGenericBase, mode=mode)
    Y, H, d = op(to_dev(Z, dtype), to_dev(V_h, dtype), to_dev(c, "f32"), to_dev(i, "f32"))
    torch.cuda.synchronize()
    return tuple(t.float().cpu().numpy() for t in (Y, H, d))


def run_low_mem(X, W, b, y0, c0, i, start=0, step=1, *, dtype="f32", mode="auto"):
    get_op()
    op = torch_native_op.make_op(native_op.LstmLowMem, mode=mode)
    Y, C, d = op(to_dev(X, dtype), to_dev(W, dtype), to_dev(b, dtype), to_dev(y0, dtype), to_dev(c0, "f32"), to_dev(i, "f32"), start, step)
    torch.cuda.synchronize()
    return tuple(t.float().cpu().numpy() for t in (Y, C, d))


def generic_base_problem(seed, T, B, n):
    rng = numpy.random.default_rng(seed)
    Z = rng.normal(0, 0.5, (T, B, 4 * n)).astype(numpy.float32)
    V = (rng.uniform(-1, 1, (n, 4 * n)) / numpy.sqrt(max(n, 1))).astype(numpy.float32)
    c = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    return Z, V, c, _holes(rng, T, B)


def low_mem_problem(seed, T, B, n_in, n):
    rng = numpy.random.default_rng(seed)
    X = rng.normal(0, 0.5, (T, B, n_in)).astype(numpy.float32)
    W = (rng.uniform(-1, 1, (n_in + n, 4 * n)) / numpy.sqrt(max(n_in + n, 1))).astype(numpy.float32)
    b = rng.normal(0, 0.2, (4 * n,)).astype(numpy.float32)
    y0 = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    c0 = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    return X, W, b, y0, c0, _holes(rng, T, B)


def test_low_mem_reference_closed_form():
    """tests/test_TFNativeOp.py:264-297: one frame, one sequence, one cell, all weights 1."""
    announce("low_mem_closed_form")
    vX, vb, vy0, vc0 = 0.2, 0.3, 0.1, 0.1
    ones = numpy.ones
    Y, C, d = run_low_mem(ones((1, 1, 1)) * vX, ones((2, 4)), ones((4,)) * vb, ones((1, 1)) * vy0, ones((1, 1)) * vc0, ones((1, 1)))
    vintern = vX + vy0 + vb
    vgates = 1.0 / (1.0 + numpy.exp(-vintern))
    vc = vgates * vc0 + vgates * numpy.tanh(vintern)
    vh = vgates * numpy.tanh(vc)
    assert Y.shape == (1, 1, 1) and C.shape == (1, 1, 1) and d.shape == (1, 1)
    assert_allclose(Y[0, 0, 0], vh, rtol=1e-6)
    assert_allclose(C[0, 0, 0], vc, rtol=1e-6)
    assert_allclose(d[0, 0], vc, rtol=1e-6)


def test_generic_base_reference_zero_run():
    """tests/test_TFNativeOp.py:234-250: zero inputs and zero state give zero output."""
    announce("generic_base_zero_run")
    T, B, n = 2, 1, 3
    z = numpy.zeros
    Y, H, d = run_generic_base(z((T, B, 4 * n)), z((n, 4 * n)), z((B, n)), numpy.ones((T, B)))
    assert Y.shape == (T, B, n) and numpy.abs(Y).max() == 0 and numpy.abs(d).max() == 0
    assert_allclose(H[:, :, n:], 0.5)
    assert numpy.abs(H[:, :, :n]).max() == 0


SHAPES = [(5, 6, 100), (1, 1, 1), (5, 3, 7), (9, 4, 33), (7, 1, 32), (6, 3, 64), (5, 17, 128), (4, 33, 64), (12, 5, 256), (40, 6, 96)]


@pytest.mark.parametrize("T,B,n", SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_generic_base_shapes(T, B, n, dtype):
    announce("generic_base_shapes", T, B, n, dtype)
    p = generic_base_problem(300 + T + B + n, T, B, n)
    want = oracle.lstm_generic_base_fwd(*p)
    _check(run_generic_base(*p, dtype=dtype), want, dtype, ("LstmGenericBase %s" % ((T, B, n),), "YHd"))


@pytest.mark.parametrize("mode", ["persistent", "graph", "stepwise"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_generic_base_modes(mode, dtype):
    T, B, n = 25, 9, 128
    announce("generic_base_modes", mode, dtype)
    p = generic_base_problem(17, T, B, n)
    want = oracle.lstm_generic_base_fwd(*p)
    _check(run_generic_base(*p, dtype=dtype, mode=mode), want, dtype, ("LstmGenericBase " + mode, "YHd"))


def test_generic_base_differs_from_native_lstm2_only_on_holes():
    """Without masked frames inside sequences and with y0 = 0 the op is NativeLstm2 (its H's first block aside)."""
    announce("generic_base_vs_native_lstm2")
    T, B, n = 11, 5, 64
    Z, V, c, _ = generic_base_problem(5, T, B, n)
    lens = numpy.array([11, 3, 7, 1, 9])
    i = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    Y, H, d = run_generic_base(Z, V, c, i)
    Y2, C2, H2, d2 = oracle.native_lstm2_fwd(Z, V, numpy.zeros((B, n), numpy.float32), c, i, 0, 1)[:4]
    assert_allclose(Y, Y2, rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(d, d2, rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(H[:, :, :n], C2, rtol=F32_RTOL, atol=F32_ATOL)
    m = i[:, :, None]  # past a sequence's end the gates see different recurrent input (zero here, the carried output there)
    assert_allclose(H[:, :, n:] * m, H2[:, :, n:] * m, rtol=F32_RTOL, atol=F32_ATOL)


LOW_MEM_SHAPES = [(5, 4, 12, 100), (1, 1, 1, 1), (5, 3, 4, 7), (6, 2, 3, 33), (7, 1, 16, 32), (6, 3, 40, 64), (5, 17, 24, 128), (12, 5, 8, 256), (30, 6, 50, 96)]


@pytest.mark.parametrize("T,B,n_in,n", LOW_MEM_SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_low_mem_shapes(T, B, n_in, n, dtype):
    announce("low_mem_shapes", T, B, n_in, n, dtype)
    p = low_mem_problem(400 + T + B + n + n_in, T, B, n_in, n)
    for start, step in [(0, 1), (0, -1), (1, 2), (1, -1), (2, -2)]:
        if start >= T or (step < 0 and T - start - 1 < start):
            continue
        want = oracle.lstm_low_mem_fwd(*p, start, step)
        got = run_low_mem(*p, start, step, dtype=dtype)
        # frames the op does not visit are unspecified in the reference (its outputs are uninitialised there)
        sl = visited_slice(T, start, step) if step > 0 else slice(T - start - 1, start - 1 if start > 0 else None, step)
        got = (got[0][sl], got[1][sl], got[2])
        want = (want[0][sl], want[1][sl], want[2])
        _check(got, want, dtype, ("LstmLowMem %s" % ((T, B, n_in, n, start, step),), "YCd"))


@pytest.mark.parametrize("mode", ["persistent", "graph", "stepwise"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_low_mem_modes(mode, dtype):
    T, B, n_in, n = 25, 9, 48, 128
    announce("low_mem_modes", mode, dtype)
    p = low_mem_problem(23, T, B, n_in, n)
    for start, step in [(0, 1), (0, -1)]:
        want = oracle.lstm_low_mem_fwd(*p, start, step)
        _check(run_low_mem(*p, start, step, dtype=dtype, mode=mode), want, dtype, ("LstmLowMem " + mode, "YCd"))


def test_low_mem_equals_native_lstm2_on_projected_input():
    """With no holes in the mask the op is NativeLstm2 on X.W_in + b with the recurrent rows of W."""
    announce("low_mem_vs_native_lstm2")
    T, B, n_in, n = 9, 4, 12, 64
    X, W, b, y0, c0, _ = low_mem_problem(31, T, B, n_in, n)
    lens = numpy.array([9, 2, 5, 9])
    i = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    Y, C, d = run_low_mem(X, W, b, y0, c0, i)
    Xp = (X.astype(numpy.float64) @ W[:n_in].astype(numpy.float64) + b).astype(numpy.float32)
    Y2, C2, _, d2 = oracle.native_lstm2_fwd(Xp, W[n_in:], y0, c0, i, 0, 1)[:4]
    # the first frame after a sequence's end still differs (y carried there vs. zero) but is masked: Y = 0, C kept
    assert_allclose(Y, Y2, rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(C, C2, rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(d, d2, rtol=F32_RTOL, atol=F32_ATOL)


def test_c_abi_errors():
    """Too small a workspace and a bad start are refused with the library's error codes; empty problems are fine."""
    announce("siblings_c_abi_errors")
    get_op()
    cabi = lib.load()
    T, B, n_in, n = 4, 2, 3, 32
    X, W, b, y0, c0, i = (to_dev(a, "f32") for a in low_mem_problem(1, T, B, n_in, n))
    Y = torch.empty((T, B, n), device="cuda:0")
    C = torch.empty((T, B, n), device="cuda:0")
    d = torch.empty((B, n), device="cuda:0")
    need = cabi.rtn_lstm_low_mem_fwd_workspace_bytes(T, B, n_in, n, lib.DTYPE_F32, 0)
    assert need > 0
    ws = torch.empty((need,), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    args = (X.data_ptr(), W.data_ptr(), b.data_ptr(), y0.data_ptr(), c0.data_ptr(), i.data_ptr())
    outs = (Y.data_ptr(), C.data_ptr(), d.data_ptr())
    rc = cabi.rtn_lstm_low_mem_fwd(*args, 0, 1, *outs, T, B, n_in, n, lib.DTYPE_F32, 0, ws.data_ptr(), need - 1, stream)
    assert rc == lib.RTN_ERR_WORKSPACE and b"workspace" in cabi.rtn_last_error()
    rc = cabi.rtn_lstm_low_mem_fwd(*args, T, 1, *outs, T, B, n_in, n, lib.DTYPE_F32, 0, ws.data_ptr(), need, stream)
    assert rc == lib.RTN_ERR_RANGE
    rc = cabi.rtn_lstm_low_mem_fwd(*args, 0, 0, *outs, T, B, n_in, n, lib.DTYPE_F32, 0, ws.data_ptr(), need, stream)
    assert rc == lib.RTN_ERR_RANGE
    rc = cabi.rtn_lstm_low_mem_fwd(*args, 2, -1, *outs, T, B, n_in, n, lib.DTYPE_F32, 0, ws.data_ptr(), need, stream)
    assert rc == lib.RTN_ERR_RANGE and b"visits no frame" in cabi.rtn_last_error()  # would run from frame 1 down to frame 2
    rc = cabi.rtn_lstm_low_mem_fwd(*args, 0, 1, *outs, T, B, n_in, n, lib.DTYPE_F32, 0, ws.data_ptr(), need, stream)
    assert rc == 0
    torch.cuda.synchronize()
    Z, V, c, i2 = (to_dev(a, "f32") for a in generic_base_problem(2, T, B, n))
    H = torch.empty((T, B, 4 * n), device="cuda:0")
    need = cabi.rtn_lstm_generic_base_fwd_workspace_bytes(T, B, n, lib.DTYPE_F32, 0)
    ws = torch.empty((need,), dtype=torch.uint8, device="cuda:0")
    gargs = (Z.data_ptr(), V.data_ptr(), c.data_ptr(), i2.data_ptr(), Y.data_ptr(), H.data_ptr(), d.data_ptr())
    rc = cabi.rtn_lstm_generic_base_fwd(*gargs, T, B, n, lib.DTYPE_F32, 0, ws.data_ptr(), need - 1, stream)
    assert rc == lib.RTN_ERR_WORKSPACE
    rc = cabi.rtn_lstm_generic_base_fwd(*gargs, T, B, n, lib.DTYPE_F32, 0, ws.data_ptr(), need, stream)
    assert rc == 0
    torch.cuda.synchronize()


def _rel_to_max(got, want):
    return float(numpy.abs(got - want).max()) / max(float(numpy.abs(want).max()), 1e-30)


GRAD_SHAPES = [(6, 7, 72), (7, 3, 16), (9, 20, 64), (6, 5, 20), (5, 2, 3), (12, 40, 128), (16, 32, 256)]


@pytest.mark.parametrize("T,B,n", GRAD_SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_generic_base_gradient(T, B, n, dtype):
    """
    ``rtn_lstm_generic_base_bwd`` against the float64 oracle of the reference's gradient code, fed the GPU's own forward
    results.  Judged like the NativeLstm2 gradient: float32 within 2e-5, bfloat16 within 2e-2 of each array's largest
    magnitude.
    """
    announce("generic_base_gradient", T, B, n, dtype)
    Z, V, c, mask = generic_base_problem(500 + T + B + n, T, B, n)
    rng = numpy.random.default_rng(600 + T + n)
    DY = rng.normal(0, 1, (T, B, n)).astype(numpy.float32)
    Dd = rng.normal(0, 1, (B, n)).astype(numpy.float32)
    get_op()
    op = torch_native_op.make_op(native_op.LstmGenericBase)
    Vd, DYd = to_dev(V, dtype), to_dev(DY, dtype)
    cd, md, Ddd = to_dev(c, "f32"), to_dev(mask, "f32"), to_dev(Dd, "f32")
    Y, H, d = op(to_dev(Z, dtype), Vd, cd, md)
    got = torch_native_op.lstm_generic_base_grad(Vd, cd, md, Y, H, DYd, Ddd)
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    want = oracle.lstm_generic_base_bwd(f(Vd), c, mask, f(Y), f(H), f(DYd), Dd, dtype=numpy.float64)
    tol = 2e-5 if dtype == "f32" else 2e-2
    for name, a, b in zip(("DZ", "DV_h", "Dc"), got, want):
        assert a.shape == b.shape and numpy.all(numpy.isfinite(f(a))), name
        assert _rel_to_max(f(a), b) <= tol, (name, _rel_to_max(f(a), b))


def test_generic_base_gradient_through_autograd():
    """LstmGenericBaseFunction under torch.autograd against autograd through a plain torch restatement (float64, CPU)."""
    announce("generic_base_autograd")
    T, B, n = 8, 5, 32
    Z, V, c, mask = generic_base_problem(77, T, B, n)
    rng = numpy.random.default_rng(78)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    ref = [torch.tensor(a.astype(numpy.float64), requires_grad=True) for a in (Z, V, c)]
    y_prev, c_prev, ys = torch.zeros((B, n), dtype=torch.float64), ref[2], []
    mt = torch.tensor(mask.astype(numpy.float64))
    for t in range(T):
        z = ref[0][t] + y_prev @ ref[1]
        g, i, fg, o = torch.tanh(z[:, :n]), torch.sigmoid(z[:, n : 2 * n]), torch.sigmoid(z[:, 2 * n : 3 * n]), torch.sigmoid(z[:, 3 * n :])
        m = mt[t][:, None]
        c_new = (c_prev * fg + g * i) * m + c_prev * (1 - m)
        y_prev, c_prev = torch.tanh(c_new) * o * m, c_new
        ys.append(y_prev)
    ((torch.stack(ys) * torch.tensor(GY)).sum() + (c_prev * torch.tensor(Gd)).sum()).backward()
    get_op()
    leaves = [to_dev(a, "f32").requires_grad_(True) for a in (Z, V, c)]
    Y, H, d = torch_native_op.LstmGenericBaseFunction.apply(*leaves, to_dev(mask, "f32"))
    assert not H.requires_grad
    ((Y * to_dev(GY, "f32")).sum() + (d * to_dev(Gd, "f32")).sum()).backward()
    torch.cuda.synchronize()
    for name, leaf, r in zip(("Z", "V_h", "c"), leaves, ref):
        assert _rel_to_max(leaf.grad.cpu().numpy().astype(numpy.float64), r.grad.numpy()) <= 2e-5, name


LOW_MEM_GRAD_SHAPES = [(6, 4, 12, 100), (5, 3, 4, 7), (7, 1, 16, 32), (6, 3, 40, 64), (9, 17, 24, 128), (12, 5, 8, 256), (1, 1, 1, 1), (8, 2, 5, 48)]


def _low_mem_grad_case(seed, T, B, n_in, n, start, step, dtype, mask=None):
    X, W, b, y0, c0, holes = low_mem_problem(seed, T, B, n_in, n)
    mask = holes if mask is None else mask
    rng = numpy.random.default_rng(seed + 1)
    DY = rng.normal(0, 1, (T, B, n)).astype(numpy.float32)
    Dd = rng.normal(0, 1, (B, n)).astype(numpy.float32)
    get_op()
    op = torch_native_op.make_op(native_op.LstmLowMem)
    Xd, Wd, bd, y0d, DYd = (to_dev(a, dtype) for a in (X, W, b, y0, DY))
    c0d, md, Ddd = to_dev(c0, "f32"), to_dev(mask, "f32"), to_dev(Dd, "f32")
    Y, C, d = op(Xd, Wd, bd, y0d, c0d, md, start, step)
    got = torch_native_op.lstm_low_mem_grad(Xd, Wd, bd, y0d, c0d, md, start, step, Y, C, DYd, Ddd)
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    want = oracle.lstm_low_mem_bwd(f(Xd), f(Wd), f(bd), f(y0d), c0, mask, start, step, f(Y), f(C), f(DYd), Dd, dtype=numpy.float64)
    return [f(a) for a in got], want


@pytest.mark.parametrize("T,B,n_in,n", LOW_MEM_GRAD_SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_low_mem_gradient(T, B, n_in, n, dtype):
    """
    ``rtn_lstm_low_mem_bwd`` against the float64 restatement of the reference's gradient code, fed the GPU's own forward
    results, with holes anywhere in the mask (on masked frames both sides follow the reference's formulas to the letter).
    Judged like the other gradients: float32 within 2e-5, bfloat16 within 3e-2 of each array's largest magnitude (the
    gates are computed again from bfloat16 products here, one rounding more than where the forward pass stored them).
    """
    announce("low_mem_gradient", T, B, n_in, n, dtype)
    tol = 2e-5 if dtype == "f32" else 3e-2
    for start, step in [(0, 1), (0, -1), (T - 1 - 2 * ((T - 1) // 2), 2), (1, -1), (0, -3)]:
        if start < 0 or start >= T:
            continue
        first, far = (start, T - 1) if step > 0 else (T - start - 1, start)
        if (step < 0 and first < far) or abs(first - far) % abs(step) != 0:
            continue
        got, want = _low_mem_grad_case(800 + T + B + n + n_in, T, B, n_in, n, start, step, dtype)
        for name, a, w in zip(("DX", "DW", "Db", "Dh", "Dc"), got, want):
            assert a.shape == w.shape and numpy.all(numpy.isfinite(a)), (name, start, step)
            assert _rel_to_max(a, w) <= tol, (name, start, step, _rel_to_max(a, w))


@pytest.mark.parametrize("kernel", [1, 2])
def test_low_mem_gradient_kernels(kernel):
    """Per-frame launches and the persistent gradient kernel give the same LstmLowMem gradients."""
    from _gpu_util import env

    announce("low_mem_gradient kernel", kernel)
    with env(RTN_LSTM2_BWD_KERNEL=kernel):
        for dtype, tol in (("f32", 2e-5), ("bf16", 3e-2)):
            got, want = _low_mem_grad_case(850, 10, 6, 20, 128, 0, -1, dtype)
            for name, a, w in zip(("DX", "DW", "Db", "Dh", "Dc"), got, want):
                assert _rel_to_max(a, w) <= tol, (name, dtype, _rel_to_max(a, w))


def test_low_mem_gradient_through_autograd():
    """LstmLowMemFunction under torch.autograd against autograd through a plain torch restatement (float64, CPU) on a
    right-padded batch, where the reference's formulas are the gradient of its forward pass."""
    announce("low_mem_autograd")
    T, B, n_in, n = 9, 5, 12, 32
    X, W, b, y0, c0, _ = low_mem_problem(860, T, B, n_in, n)
    lens = numpy.array([9, 4, 7, 1, 9])
    mask = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    rng = numpy.random.default_rng(861)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    ref = [torch.tensor(a.astype(numpy.float64), requires_grad=True) for a in (X, W, b, y0, c0)]
    mt = torch.tensor(mask.astype(numpy.float64))
    y_prev, c_prev, ys = ref[3], ref[4], []
    for t in range(T):
        z = torch.cat([ref[0][t], y_prev], dim=1) @ ref[1] + ref[2]
        g, i, fg, o = torch.tanh(z[:, :n]), torch.sigmoid(z[:, n : 2 * n]), torch.sigmoid(z[:, 2 * n : 3 * n]), torch.sigmoid(z[:, 3 * n :])
        m = mt[t][:, None]
        c_new = (c_prev * fg + g * i) * m + c_prev * (1 - m)
        y_prev, c_prev = torch.tanh(c_new) * o * m, c_new
        ys.append(y_prev)
    ((torch.stack(ys) * torch.tensor(GY)).sum() + (c_prev * torch.tensor(Gd)).sum()).backward()
    get_op()
    leaves = [to_dev(a, "f32").requires_grad_(True) for a in (X, W, b, y0, c0)]
    Y, C, d = torch_native_op.LstmLowMemFunction.apply(*leaves, to_dev(mask, "f32"), 0, 1)
    assert not C.requires_grad
    ((Y * to_dev(GY, "f32")).sum() + (d * to_dev(Gd, "f32")).sum()).backward()
    torch.cuda.synchronize()
    for name, leaf, r in zip(("X", "W", "b", "y0", "c0"), leaves, ref):
        assert _rel_to_max(leaf.grad.cpu().numpy().astype(numpy.float64), r.grad.numpy()) <= 2e-5, name


def test_low_mem_gradient_refusals():
    announce("low_mem_gradient refusals")
    get_op()
    T, B, n_in, n = 8, 2, 4, 32
    z = lambda *s: torch.zeros(*s, device="cuda:0")  # noqa: E731
    args = lambda start, step: (z(T, B, n_in), z(n_in + n, 4 * n), z(4 * n), z(B, n), z(B, n), z(T, B), start, step, z(T, B, n), z(T, B, n), z(T, B, n), z(B, n))  # noqa: E731
    for start, step in ((0, 2), (2, 3), (1, -4)):
        with pytest.raises(RuntimeError, match="stride"):
            torch_native_op.lstm_low_mem_grad(*args(start, step))
    with pytest.raises(RuntimeError, match="visits no frame"):
        torch_native_op.lstm_low_mem_grad(*args(6, -1))
    with pytest.raises(RuntimeError, match="step must not be 0"):
        torch_native_op.lstm_low_mem_grad(*args(0, 0))
    cabi = lib.load()
    assert cabi.rtn_lstm_low_mem_bwd_workspace_bytes(T, B, n_in, n, lib.DTYPE_F32) > cabi.rtn_native_lstm2_bwd_workspace_bytes(T, B, n, lib.DTYPE_F32)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_sibling_ops_recorded_into_a_callers_graph(dtype):
    """LstmLowMem (whose input projection is a rocBLAS GEMM) and LstmGenericBase with its gradient under stream capture,
    after one eager run: recorded into the caller's graph, replayed twice with new inputs, equal to the eager results
    (bit for bit in the forward pass, up to rounding in the gradient, which takes another decomposition)."""
    announce("siblings captured", dtype)
    get_op()
    T, B, n_in, n = 9, 6, 24, 64
    lm = torch_native_op.make_op(native_op.LstmLowMem)
    gb = torch_native_op.make_op(native_op.LstmGenericBase)
    lm_problems = [low_mem_problem(700 + k, T, B, n_in, n) for k in range(2)]
    gb_problems = [generic_base_problem(710 + k, T, B, n) for k in range(2)]
    rng = numpy.random.default_rng(3)
    DYs = [rng.normal(0, 1, (T, B, n)).astype(numpy.float32) for _ in range(2)]
    Dds = [rng.normal(0, 1, (B, n)).astype(numpy.float32) for _ in range(2)]
    X, W, b, y0, c0, i = lm_problems[0]
    lm_in = [to_dev(X, dtype), to_dev(W, dtype), to_dev(b, dtype), to_dev(y0, dtype), to_dev(c0, "f32"), to_dev(i, "f32")]
    Z, V, c, ig = gb_problems[0]
    gb_in = [to_dev(Z, dtype), to_dev(V, dtype), to_dev(c, "f32"), to_dev(ig, "f32")]
    DYd, Ddd = to_dev(DYs[0], dtype), to_dev(Dds[0], "f32")

    def step():
        lm_out = lm(*lm_in, 0, 1)
        Y, H, d = gb(*gb_in)
        grads = torch_native_op.lstm_generic_base_grad(gb_in[1], gb_in[2], gb_in[3], Y, H, DYd, Ddd)
        return list(lm_out) + [Y, H, d], list(grads)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        fwd_out, grad_out = step()
    for k in range(2):
        for dst, src in zip(lm_in, lm_problems[k]):
            dst.copy_(to_dev(src, "f32" if dst.dtype == torch.float32 else dtype))
        for dst, src in zip(gb_in, gb_problems[k]):
            dst.copy_(to_dev(src, "f32" if dst.dtype == torch.float32 else dtype))
        DYd.copy_(to_dev(DYs[k], dtype))
        Ddd.copy_(to_dev(Dds[k], "f32"))
        graph.replay()
        torch.cuda.synchronize()
        got_f = [t.clone() for t in fwd_out]
        got_g = [t.clone() for t in grad_out]
        eager_f, eager_g = step()
        torch.cuda.synchronize()
        for idx, (a, e) in enumerate(zip(got_f, eager_f)):
            assert torch.equal(a, e), (k, "forward output", idx)
        for idx, (a, e) in enumerate(zip(got_g, eager_g)):
            scale = max(float(e.float().abs().max()), 1e-30)
            assert float((a.float() - e.float()).abs().max()) / scale <= (2e-5 if dtype == "f32" else 2e-2), (k, "gradient", idx)
