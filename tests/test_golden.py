"""
The committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from the textbook LSTM and
torch.nn.LSTM in float64 -- nothing of oracle/ or of the HIP library) against the CPU oracle here and, under ``-m gpu``,
against the HIP path through the C ABI.  The vectors are data: a change of the oracle, of the textbook helpers or of the
kernels cannot move them.
"""

from __future__ import annotations

import os

import numpy
import pytest
from numpy.testing import assert_allclose

from oracle import lstm2_oracle as oracle
from _textbook import REFERENCE_START_STEP, visited_slice

_golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with numpy.load(os.path.join(_golden, name + ".npz"), allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def _tag(start, step):
    return "s%i_%s%i" % (start, "p" if step > 0 else "m", abs(step))


@pytest.mark.parametrize("start,step", REFERENCE_START_STEP)
def test_oracle_reference_fixture(start, step):
    """The reference's fixture with its comparison rules (tests/test_TFNativeOp.py:851-854): visited, unmasked frames."""
    g = load("reference_fixture")
    Y, C, H, d, y_last = oracle.native_lstm2_fwd(g["X"], g["W_r"], g["h_0"], g["c_0"], g["mask"], start, step, dtype=numpy.float64)
    sl, m = visited_slice(3, start, step), g["mask"][:, :, None]
    assert_allclose(Y[sl] * m[sl], g["h_" + _tag(start, step)][sl] * m[sl], rtol=1e-12, atol=1e-14)
    assert_allclose(C[sl] * m[sl], g["c_" + _tag(start, step)][sl] * m[sl], rtol=1e-12, atol=1e-14)
    assert_allclose(d, g["cT_" + _tag(start, step)], rtol=1e-12, atol=1e-14)
    assert_allclose(y_last, g["hT_" + _tag(start, step)], rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize("reverse", [False, True])
def test_oracle_torch_ragged(reverse):
    g = load("torch_ragged")
    tag, step = ("rev", -1) if reverse else ("fwd", 1)
    lens = g["lens"].astype(numpy.int64)
    mask = (numpy.arange(g["X"].shape[0])[:, None] < lens[None, :]).astype(numpy.float64)
    Y, C, H, d, y_last = oracle.native_lstm2_fwd(g["X"], g["W"], g["y0"], g["c0"], mask, 0, step, dtype=numpy.float64)
    assert_allclose(Y, g["Y_" + tag], rtol=1e-10, atol=1e-12)
    assert_allclose(d, g["cT_" + tag], rtol=1e-10, atol=1e-12)
    assert_allclose(y_last, g["hT_" + tag], rtol=1e-10, atol=1e-12)
    got = oracle.native_lstm2_bwd(g["X"], g["W"], g["y0"], g["c0"], mask, 0, step, Y, C, H, g["GY"], g["Gd"], dtype=numpy.float64)
    for name, a in zip(("DX", "DW", "Dy0", "Dc0"), got):
        assert_allclose(a, g["%s_%s" % (name, tag)], rtol=1e-9, atol=1e-11, err_msg=name)


def test_oracle_low_mem_closed_form():
    g = load("low_mem_closed_form")
    Y, C, d = oracle.lstm_low_mem_fwd(g["X"], g["W"], g["b"], g["y0"], g["c0"], numpy.ones((1, 1)), 0, 1, dtype=numpy.float64)
    assert_allclose(Y, g["Y"], rtol=1e-12)
    assert_allclose(C, g["C"], rtol=1e-12)
    assert_allclose(d, g["C"][0], rtol=1e-12)


# ---- the HIP path against the same vectors -------------------------------------------------------------------------------


@pytest.mark.gpu
@pytest.mark.parametrize("start,step", REFERENCE_START_STEP)
def test_gpu_reference_fixture(start, step):
    from _gpu_util import announce, run_op

    announce("golden reference_fixture", start, step)
    g = load("reference_fixture")
    Y, C, H, d, y_last = run_op(g["X"], g["W_r"], g["h_0"], g["c_0"], g["mask"], start, step)
    sl, m = visited_slice(3, start, step), g["mask"][:, :, None]
    assert_allclose(Y[sl] * m[sl], g["h_" + _tag(start, step)][sl] * m[sl], rtol=1e-5, atol=1e-6)
    assert_allclose(C[sl] * m[sl], g["c_" + _tag(start, step)][sl] * m[sl], rtol=1e-5, atol=1e-6)
    assert_allclose(d, g["cT_" + _tag(start, step)], rtol=1e-5, atol=1e-6)
    assert_allclose(y_last, g["hT_" + _tag(start, step)], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("reverse", [False, True])
def test_gpu_torch_ragged_forward_and_gradient(reverse):
    """float32 on the GPU against torch.nn.LSTM in float64: outputs to 1e-5 relative (2e-6 absolute near zero), gradients
    within 2e-5 of each array's largest magnitude."""
    import torch

    from returnn_amd import torch_native_op
    from _gpu_util import announce, get_op, to_dev

    announce("golden torch_ragged", reverse)
    g = load("torch_ragged")
    tag, step = ("rev", -1) if reverse else ("fwd", 1)
    lens = g["lens"].astype(numpy.int64)
    mask = (numpy.arange(g["X"].shape[0])[:, None] < lens[None, :]).astype(numpy.float32)
    get_op()
    leaves = [to_dev(g[k], "f32").requires_grad_(True) for k in ("X", "W", "y0", "c0")]
    Y, C, H, d = torch_native_op.NativeLstm2Function.apply(*leaves, to_dev(mask, "f32"), 0, step)
    ((Y * to_dev(g["GY"], "f32")).sum() + (d * to_dev(g["Gd"], "f32")).sum()).backward()
    torch.cuda.synchronize()
    assert_allclose(Y.detach().cpu().numpy(), g["Y_" + tag], rtol=1e-5, atol=2e-6)
    assert_allclose(d.detach().cpu().numpy(), g["cT_" + tag], rtol=1e-5, atol=2e-6)
    for name, leaf in zip(("DX", "DW", "Dy0", "Dc0"), leaves):
        want = g["%s_%s" % (name, tag)]
        err = numpy.abs(leaf.grad.cpu().numpy() - want).max() / numpy.abs(want).max()
        assert err <= 2e-5, (name, err)


@pytest.mark.gpu
def test_gpu_low_mem_closed_form():
    import torch

    from returnn_amd import native_op, torch_native_op
    from _gpu_util import announce, get_op, to_dev

    announce("golden low_mem_closed_form")
    g = load("low_mem_closed_form")
    get_op()
    op = torch_native_op.make_op(native_op.LstmLowMem)
    Y, C, d = op(*(to_dev(g[k], "f32") for k in ("X", "W", "b", "y0", "c0")), torch.ones((1, 1), device="cuda:0"), 0, 1)
    torch.cuda.synchronize()
    assert_allclose(Y.cpu().numpy(), g["Y"], rtol=1e-6)
    assert_allclose(C.cpu().numpy(), g["C"], rtol=1e-6)
    assert_allclose(d.cpu().numpy(), g["C"][0], rtol=1e-6)
