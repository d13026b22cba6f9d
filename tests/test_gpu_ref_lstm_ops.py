"""
The reference's own source of the three LSTM ops (``NativeLstm2``, ``LstmGenericBase``, ``LstmLowMem``: ``c_fw_code``,
``c_bw_code`` and kernels as they stand in returnn/native_op.py), compiled for gfx950 by this package's op loader together
with the gradient ops the loader derives for them, run on the GPU against

* the committed golden vectors (tests/golden/: the reference's fixture with its comparison rules, a ragged batch with
  gradients from torch autograd in float64, the one-cell LstmLowMem closed form),
* the CPU oracle on seeded problems, and
* this package's hand-written kernels on the same inputs.

The shared objects are built where the reference tree is (``python tests/build_ref_ops.py``, also part of the build
step) into ``tests/_built_ref_ops/``; here they are only loaded.  What runs is the reference's op code against this
package's support header (arrays, launches, ``affine_raw`` on rocBLAS) -- a check of the loader and of the derived
gradient descriptions on the ops this package is about, and a second, independently written implementation next to the
hand-written kernels; it is not the oracle.
"""

from __future__ import annotations

import json
import os

import numpy
import pytest
import torch
from numpy.testing import assert_allclose

from oracle import lstm2_oracle as oracle
from returnn_amd import native_op, op_loader, torch_native_op
from _gpu_util import announce, random_problem, run_op
from _textbook import REFERENCE_START_STEP, visited_slice
from test_golden import _tag, load

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OPS_DIR = os.path.join(ROOT, "tests", "_built_ref_ops")


def _have(name):
    path = os.path.join(OPS_DIR, "ops.json")
    return os.path.exists(path) and name in json.load(open(path)) and os.path.exists(os.path.join(OPS_DIR, name + ".so"))


needs_ops = pytest.mark.skipif(
    not all(_have(n) for n in ("NativeLstm2", "GradOfNativeLstm2", "LstmGenericBase", "GradOfLstmGenericBase", "LstmLowMem", "GradOfLstmLowMem")),
    reason="tests/_built_ref_ops lacks the LSTM ops (python tests/build_ref_ops.py, where the reference tree is)",
)


def _op(name):
    table = json.load(open(os.path.join(OPS_DIR, "ops.json")))
    return op_loader.CompiledOp.from_shared_object(name, table[name]["in_info"], table[name]["out_info"], os.path.join(OPS_DIR, name + ".so"))


def _dev(a):
    return torch.from_numpy(numpy.ascontiguousarray(a, dtype=numpy.float32)).to("cuda:0")


def _np(t):
    return t.detach().float().cpu().numpy()


def _rel(got, want):
    return float(numpy.abs(got - want).max()) / max(float(numpy.abs(want).max()), 1e-30)


@needs_ops
@pytest.mark.parametrize("start,step", REFERENCE_START_STEP)
def test_reference_native_lstm2_source_on_the_reference_fixture(start, step):
    announce("reference source NativeLstm2, fixture", start, step)
    g = load("reference_fixture")
    op = _op("NativeLstm2")
    Y, C, H, d = (_np(t) for t in op(_dev(g["X"]), _dev(g["W_r"]), _dev(g["h_0"]), _dev(g["c_0"]), _dev(g["mask"]), start, step))
    torch.cuda.synchronize()
    sl, m = visited_slice(3, start, step), g["mask"][:, :, None]
    assert_allclose(Y[sl] * m[sl], g["h_" + _tag(start, step)][sl] * m[sl], rtol=1e-5, atol=1e-6)
    assert_allclose(C[sl] * m[sl], g["c_" + _tag(start, step)][sl] * m[sl], rtol=1e-5, atol=1e-6)
    assert_allclose(d, g["cT_" + _tag(start, step)], rtol=1e-5, atol=1e-6)
    # the hand-written kernels on the same inputs: every output, H and the unvisited frames included
    mine = run_op(g["X"], g["W_r"], g["h_0"], g["c_0"], g["mask"], start, step)
    for name, a, b in zip("YCHd", (Y, C, H, d), mine):
        assert_allclose(a, b, rtol=1e-5, atol=1e-6, err_msg=name)


@needs_ops
@pytest.mark.parametrize("T,B,n,start,step", [(12, 5, 24, 0, 1), (12, 5, 24, 1, -1), (9, 3, 64, 0, -1), (7, 20, 128, 2, 2), (6, 4, 100, 0, 1)])
def test_reference_native_lstm2_source_against_oracle_and_kernels(T, B, n, start, step):
    announce("reference source NativeLstm2", T, B, n, start, step)
    X, W, y0, c0, i = random_problem(700 + T + n, T, B, n)
    op = _op("NativeLstm2")
    got = [_np(t) for t in op(_dev(X), _dev(W), _dev(y0), _dev(c0), _dev(i), start, step)]
    torch.cuda.synchronize()
    want = oracle.native_lstm2_fwd(X, W, y0, c0, i, start, step, dtype=numpy.float64)[:4]
    mine = run_op(X, W, y0, c0, i, start, step)[:4]
    for name, a, b, c in zip("YCHd", got, want, mine):
        assert_allclose(a, b, rtol=1e-5, atol=2e-6, err_msg="reference source against the oracle: " + name)
        assert_allclose(c, a, rtol=1e-5, atol=2e-6, err_msg="kernels against the reference source: " + name)


@needs_ops
@pytest.mark.parametrize("reverse", [False, True])
def test_reference_native_lstm2_gradient_source_on_the_ragged_golden_batch(reverse):
    """Forward and derived gradient op from the reference's source against gradients of torch autograd in float64."""
    announce("reference source GradOfNativeLstm2, ragged golden batch", reverse)
    g = load("torch_ragged")
    tag, step = ("rev", -1) if reverse else ("fwd", 1)
    T = g["X"].shape[0]
    mask = (numpy.arange(T)[:, None] < g["lens"].astype(numpy.int64)[None, :]).astype(numpy.float32)
    ins = [_dev(g[k]) for k in ("X", "W", "y0", "c0")] + [_dev(mask)]
    Y, C, H, d = _op("NativeLstm2")(*ins, 0, step)
    assert_allclose(_np(Y), g["Y_" + tag], rtol=1e-5, atol=2e-6)
    assert_allclose(_np(d), g["cT_" + tag], rtol=1e-5, atol=2e-6)
    DX, DW, Dy0, Dc0 = _op("GradOfNativeLstm2")(*ins, 0, step, Y, C, H, _dev(g["GY"]), _dev(g["Gd"]))
    torch.cuda.synchronize()
    mine = torch_native_op.native_lstm2_grad(ins[1], ins[2], ins[3], ins[4], 0, step, Y, C, H, _dev(g["GY"]), _dev(g["Gd"]))
    torch.cuda.synchronize()
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), (DX, DW, Dy0, Dc0), mine):
        assert _rel(_np(a), g["%s_%s" % (name, tag)]) <= 2e-5, name
        assert _rel(_np(b), _np(a)) <= 2e-5, "kernels against the reference source: " + name


@needs_ops
@pytest.mark.parametrize("T,B,n,start,step", [(8, 4, 24, 0, 1), (8, 4, 24, 1, -1), (7, 6, 64, 0, -2)])
def test_reference_native_lstm2_gradient_source_against_oracle(T, B, n, start, step):
    announce("reference source GradOfNativeLstm2", T, B, n, start, step)
    X, W, y0, c0, i = random_problem(800 + T + n, T, B, n)
    rng = numpy.random.default_rng(5)
    DY = rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32)
    Dd = rng.normal(0, 1.0, (B, n)).astype(numpy.float32)
    ins = [_dev(a) for a in (X, W, y0, c0, i)]
    Y, C, H, d = _op("NativeLstm2")(*ins, start, step)
    got = _op("GradOfNativeLstm2")(*ins, start, step, Y, C, H, _dev(DY), _dev(Dd))
    torch.cuda.synchronize()
    f = lambda t: _np(t).astype(numpy.float64)  # noqa: E731
    want = oracle.native_lstm2_bwd(X, W, y0, c0, i, start, step, f(Y), f(C), f(H), DY, Dd, dtype=numpy.float64)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert _rel(_np(a), b) <= 2e-5, name


@needs_ops
def test_reference_lstm_low_mem_source():
    announce("reference source LstmLowMem")
    g = load("low_mem_closed_form")
    op = _op("LstmLowMem")
    one = numpy.ones((1, 1), dtype=numpy.float32)
    Y, C, d = (_np(t) for t in op(_dev(g["X"]), _dev(g["W"]), _dev(g["b"]), _dev(g["y0"]), _dev(g["c0"]), _dev(one), 0, 1))
    assert_allclose(Y, g["Y"], rtol=1e-6)
    assert_allclose(C, g["C"], rtol=1e-6)
    assert_allclose(d, g["C"][0], rtol=1e-6)
    # seeded problems with ragged lengths against the oracle and this package's entry; then the derived gradient op
    for T, B, n_in, n, start, step in [(9, 4, 12, 16, 0, 1), (7, 5, 40, 64, 0, -1)]:
        rng = numpy.random.default_rng(T + n)
        X = rng.normal(0, 0.5, (T, B, n_in)).astype(numpy.float32)
        W = (rng.uniform(-1, 1, (n_in + n, 4 * n)) / numpy.sqrt(n_in + n)).astype(numpy.float32)
        b = rng.normal(0, 0.1, (4 * n,)).astype(numpy.float32)
        y0, c0 = (rng.normal(0, 0.3, (B, n)).astype(numpy.float32) for _ in range(2))
        i = numpy.ones((T, B), dtype=numpy.float32)  # (the gradient of this op is only defined without holes behind valid frames)
        ins = [_dev(a) for a in (X, W, b, y0, c0, i)]
        Y, C, d = op(*ins, start, step)
        torch.cuda.synchronize()
        want = oracle.lstm_low_mem_fwd(X, W, b, y0, c0, i, start, step, dtype=numpy.float64)
        for name, a, w in zip("YCd", (Y, C, d), want):
            assert_allclose(_np(a), w, rtol=1e-5, atol=2e-6, err_msg=name)
        mine = torch_native_op.make_op(native_op.LstmLowMem)(*ins, start, step)
        for name, a, m in zip("YCd", (Y, C, d), mine):
            assert_allclose(_np(m), _np(a), rtol=1e-5, atol=2e-6, err_msg="kernels against the reference source: " + name)
        DY = _dev(rng.normal(0, 1.0, (T, B, n)))
        Dd = _dev(rng.normal(0, 1.0, (B, n)))
        got = _op("GradOfLstmLowMem")(*ins, start, step, Y, C, DY, Dd)
        torch.cuda.synchronize()
        f = lambda t: _np(t).astype(numpy.float64)  # noqa: E731
        wantg = oracle.lstm_low_mem_bwd(X, W, b, y0, c0, i, start, step, f(Y), f(C), f(DY), f(Dd), dtype=numpy.float64)
        for name, a, w in zip(("DX", "DW", "Db", "Dh", "Dc"), got, wantg):
            assert _rel(_np(a), w) <= 3e-5, name


@needs_ops
@pytest.mark.parametrize("T,B,n", [(9, 4, 16), (7, 5, 64)])
def test_reference_lstm_generic_base_source(T, B, n):
    announce("reference source LstmGenericBase", T, B, n)
    rng = numpy.random.default_rng(900 + T + n)
    Z = rng.normal(0, 0.5, (T, B, 4 * n)).astype(numpy.float32)
    V = (rng.uniform(-1, 1, (n, 4 * n)) / numpy.sqrt(n)).astype(numpy.float32)
    c = rng.normal(0, 0.3, (B, n)).astype(numpy.float32)
    lens = rng.integers(1, T + 1, size=(B,))
    lens[0] = T
    i = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    Y, H, d = _op("LstmGenericBase")(_dev(Z), _dev(V), _dev(c), _dev(i))
    torch.cuda.synchronize()
    want = oracle.lstm_generic_base_fwd(Z, V, c, i, dtype=numpy.float64)
    for name, a, w in zip("YHd", (Y, H, d), want):
        assert_allclose(_np(a), w, rtol=1e-5, atol=2e-6, err_msg=name)
    DY = rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32)
    Dd = rng.normal(0, 1.0, (B, n)).astype(numpy.float32)
    f = lambda t: _np(t).astype(numpy.float64)  # noqa: E731
    wantg = oracle.lstm_generic_base_bwd(V, c, i, f(Y), f(H), DY, Dd, dtype=numpy.float64)
    # (the reference's gradient code works in place on H and on the error of Y: it gets copies)
    got = _op("GradOfLstmGenericBase")(_dev(V), _dev(c), _dev(i), Y, H.clone(), _dev(DY), _dev(Dd))
    torch.cuda.synchronize()
    for name, a, w in zip(("DZ", "DV_h", "Dc"), got[:3], wantg):
        assert _rel(_np(a), w) <= 2e-5, name
