"""
Pins the CPU oracle of the NativeLstm2 gradient op (oracle/lstm2_oracle_bwd.c) with things its code does not contain:
autograd through ``torch.nn.LSTM`` (float64; full-length and packed ragged batches, both directions, initial states,
error signals on Y and on the final cell), central finite differences of the already pinned forward oracle for every
differentiable input (including start/step variants that skip frames), and a closed form for a single cell.
The reference checks its gradient op the same way, against the framework's own gradients of an unrolled LSTM
(tests/test_TFNativeOp.py:909-1161).
"""

from __future__ import annotations

import numpy
import pytest
import torch
from numpy.testing import assert_allclose

from oracle import lstm2_oracle as oracle
from _textbook import torch_lstm_grads  # noqa: F401  (other tests import it from here)
from _textbook import sigmoid


def _problem(seed, T, B, n, ragged=True):
    rng = numpy.random.default_rng(seed)
    X = rng.normal(0, 0.7, (T, B, 4 * n))
    W = rng.normal(0, 0.5, (n, 4 * n))
    y0 = rng.normal(0, 0.4, (B, n))
    c0 = rng.normal(0, 0.4, (B, n))
    lens = rng.integers(1, T + 1, size=(B,)) if ragged else numpy.full((B,), T)
    lens[0] = T
    mask = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float64)
    GY = rng.normal(0, 1.0, (T, B, n))
    Gd = rng.normal(0, 1.0, (B, n))
    return X, W, y0, c0, mask, lens, GY, Gd


def _oracle_grads(X, W, y0, c0, mask, start, step, GY, Gd, dtype=numpy.float64):
    Y, C, H, d, _ = oracle.native_lstm2_fwd(X, W, y0, c0, mask, start, step, dtype=dtype)
    return oracle.native_lstm2_bwd(X, W, y0, c0, mask, start, step, Y, C, H, GY, Gd, dtype=dtype)


@pytest.mark.parametrize("ragged", [False, True])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("T,B,n", [(1, 1, 1), (6, 4, 5), (11, 3, 8)])
def test_bwd_vs_torch_autograd(T, B, n, ragged, reverse):
    X, W, y0, c0, mask, lens, GY, Gd = _problem(T * 7 + n, T, B, n, ragged)
    want = torch_lstm_grads(X, W, y0, c0, lens, reverse, GY, Gd)
    GY_dirty = GY + 3.0 * (1.0 - mask)[:, :, None]  # error signals on padded frames must not matter
    got = _oracle_grads(X, W, y0, c0, mask, 0, -1 if reverse else 1, GY_dirty, Gd)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert_allclose(a, b, rtol=1e-9, atol=1e-11, err_msg=name)


def _loss(X, W, y0, c0, mask, start, step, GY, Gd):
    Y, C, H, d, _ = oracle.native_lstm2_fwd(X, W, y0, c0, mask, start, step, dtype=numpy.float64)
    return float((Y * GY).sum() + (d * Gd).sum())


@pytest.mark.parametrize("start,step", [(0, 1), (0, -1), (2, 1), (1, -1), (0, 2), (1, -3), (4, 5)])
def test_bwd_vs_finite_differences(start, step):
    T, B, n = 7, 3, 4
    X, W, y0, c0, mask, lens, GY, Gd = _problem(start * 5 + step + 50, T, B, n)
    got = dict(zip(("X", "W", "y0", "c0"), _oracle_grads(X, W, y0, c0, mask, start, step, GY, Gd)))
    args = {"X": X, "W": W, "y0": y0, "c0": c0}
    eps = 1e-6
    rng = numpy.random.default_rng(1)
    for name, arr in args.items():
        flat = arr.reshape(-1)
        idxs = rng.choice(flat.size, size=min(flat.size, 60), replace=False)
        for idx in idxs:
            old = flat[idx]
            flat[idx] = old + eps
            lp = _loss(args["X"], args["W"], args["y0"], args["c0"], mask, start, step, GY, Gd)
            flat[idx] = old - eps
            lm = _loss(args["X"], args["W"], args["y0"], args["c0"], mask, start, step, GY, Gd)
            flat[idx] = old
            num = (lp - lm) / (2 * eps)
            assert abs(num - got[name].reshape(-1)[idx]) <= 1e-6 * max(1.0, abs(num)), (name, idx, num, got[name].reshape(-1)[idx])


def test_bwd_unvisited_and_masked_frames_get_zero():
    T, B, n = 9, 3, 4
    X, W, y0, c0, mask, lens, GY, Gd = _problem(3, T, B, n)
    DX, DW, Dy0, Dc0 = _oracle_grads(X, W, y0, c0, mask, 1, 3, GY, Gd)
    visited = numpy.zeros(T, bool)
    visited[1::3] = True
    assert numpy.abs(DX[~visited]).max() == 0.0
    assert numpy.abs(DX * (1.0 - mask)[:, :, None]).max() == 0.0
    assert numpy.abs(DX[visited] * mask[visited][:, :, None]).max() > 0.0


def test_bwd_closed_form_single_cell():
    """T=B=n=1: every derivative written out by hand."""
    x = numpy.array([0.3, -0.2, 0.5, 0.1])  # cell-in, input, forget, output
    w = numpy.array([0.7, -0.4, 0.2, 0.6])
    y0, c0, gy, gd = 0.5, -0.8, 1.3, -0.6
    z = x + y0 * w
    g, i, f, o = numpy.tanh(z[0]), sigmoid(z[1]), sigmoid(z[2]), sigmoid(z[3])
    c = f * c0 + g * i
    tc = numpy.tanh(c)
    dc = gd + gy * o * (1 - tc * tc)
    dz = numpy.array([dc * i * (1 - g * g), dc * g * i * (1 - i), dc * c0 * f * (1 - f), gy * tc * o * (1 - o)])
    DX, DW, Dy0, Dc0 = _oracle_grads(x.reshape(1, 1, 4), w.reshape(1, 4), numpy.array([[y0]]), numpy.array([[c0]]),
                                     numpy.ones((1, 1)), 0, 1, numpy.array([[[gy]]]), numpy.array([[gd]]))  # fmt: skip
    assert_allclose(DX.reshape(4), dz, rtol=1e-12)
    assert_allclose(DW.reshape(4), y0 * dz, rtol=1e-12)
    assert_allclose(Dy0.reshape(()), (dz * w).sum(), rtol=1e-12)
    assert_allclose(Dc0.reshape(()), dc * f, rtol=1e-12)


def test_bwd_zero_length_and_float32():
    B, n = 2, 3
    z = numpy.zeros
    DX, DW, Dy0, Dc0 = oracle.native_lstm2_bwd(z((0, B, 4 * n)), z((n, 4 * n)), z((B, n)), z((B, n)), z((0, B)), 0, 1,
                                               z((0, B, n)), z((0, B, n)), z((0, B, 4 * n)), z((0, B, n)),
                                               numpy.ones((B, n)), dtype=numpy.float64)  # fmt: skip
    assert DX.shape == (0, B, 4 * n) and numpy.abs(DW).max() == 0 and numpy.abs(Dy0).max() == 0 and (Dc0 == 1).all()
    X, W, y0, c0, mask, lens, GY, Gd = _problem(9, 8, 4, 6)
    g64 = _oracle_grads(X, W, y0, c0, mask, 0, 1, GY, Gd, dtype=numpy.float64)
    g32 = _oracle_grads(X, W, y0, c0, mask, 0, 1, GY, Gd, dtype=numpy.float32)
    for a, b in zip(g32, g64):
        assert a.dtype == numpy.float32
        assert_allclose(a, b, rtol=2e-4, atol=2e-5)
    with pytest.raises(ValueError):
        _oracle_grads(X, W, y0, c0, mask, 8, 1, GY, Gd)


@pytest.mark.parametrize("start,step", [(0, 1), (0, -1), (1, 2), (2, -3)])
def test_bwd_blas_variant_equals_the_restatement(start, step):
    """The BLAS-structured variant that the benchmark times computes the same thing."""
    X, W, y0, c0, mask, lens, GY, Gd = _problem(17, 10, 5, 12)
    Y, C, H, d, _ = oracle.native_lstm2_fwd(X, W, y0, c0, mask, start, step, dtype=numpy.float32)
    want = oracle.native_lstm2_bwd(X, W, y0, c0, mask, start, step, Y, C, H, GY, Gd, dtype=numpy.float32)
    got = oracle.native_lstm2_bwd_blas(W, y0, c0, mask, start, step, Y, C, H, GY, Gd)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert_allclose(a, b, rtol=1e-4, atol=1e-5, err_msg=name)
