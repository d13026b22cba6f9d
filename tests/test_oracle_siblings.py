"""
Pins the CPU oracle of the sibling ops (oracle/lstm_siblings_oracle.c): the reference's own closed-form vector for
LstmLowMem (tests/test_TFNativeOp.py:264-297), its all-zero run of the LstmGenericBase cell (:234-250), an independently
written float64 loop that has masked frames in the middle of sequences (where these ops differ from NativeLstm2: the
recurrent input is the masked output of the frame before, not the last valid output), torch.nn.LSTM on full-length
batches, and the NativeLstm2 oracle wherever the semantics coincide.
"""

from __future__ import annotations

import numpy
import pytest
from numpy.testing import assert_allclose

from oracle import lstm2_oracle as oracle
from _textbook import sigmoid, torch_lstm


def _loop(Xp, W_rec, y0, c0, mask, frames):
    """Plain float64 recurrence over `frames` with 'output of the frame before' as recurrent input."""
    T, B, n4 = Xp.shape
    n = n4 // 4
    Y = numpy.zeros((T, B, n))
    C = numpy.zeros((T, B, n))
    G = numpy.zeros((T, B, 4 * n))
    y_prev, c_prev = y0, c0
    for t in frames:
        z = Xp[t] + y_prev @ W_rec
        g, i, f, o = numpy.tanh(z[:, :n]), sigmoid(z[:, n : 2 * n]), sigmoid(z[:, 2 * n : 3 * n]), sigmoid(z[:, 3 * n :])
        m = mask[t][:, None]
        c = (c_prev * f + g * i) * m + c_prev * (1 - m)
        y = numpy.tanh(c) * o * m
        Y[t], C[t] = y, c
        G[t] = numpy.concatenate([c, i, f, o], axis=1)
        y_prev, c_prev = y, c
    return Y, C, G, c_prev


def _random(seed, T, B, n, n_in=None):
    rng = numpy.random.default_rng(seed)
    Z = rng.normal(0, 0.8, (T, B, 4 * n))
    V = rng.normal(0, 0.5, (n, 4 * n))
    c0 = rng.normal(0, 0.5, (B, n))
    y0 = rng.normal(0, 0.5, (B, n))
    mask = (rng.random((T, B)) > 0.3).astype(numpy.float64)  # holes anywhere
    out = dict(Z=Z, V=V, c0=c0, y0=y0, mask=mask)
    if n_in is not None:
        out["X"] = rng.normal(0, 0.8, (T, B, n_in))
        out["W"] = rng.normal(0, 0.5, (n_in + n, 4 * n))
        out["b"] = rng.normal(0, 0.3, (4 * n,))
    return out


def test_low_mem_reference_closed_form():
    """tests/test_TFNativeOp.py:264-297 (test_LstmLowMem_fwd_simple_1), same numbers, same expectations."""
    vX, vb, vy0, vc0 = 0.2, 0.3, 0.1, 0.1
    X = numpy.ones((1, 1, 1)) * vX
    W = numpy.ones((2, 4))
    b = numpy.ones((4,)) * vb
    Y, C, d = oracle.lstm_low_mem_fwd(X, W, b, numpy.ones((1, 1)) * vy0, numpy.ones((1, 1)) * vc0, numpy.ones((1, 1)), 0, 1)
    vintern = vX + vy0 + vb
    vcellIn = numpy.tanh(vintern)
    vgates = 1.0 / (1.0 + numpy.exp(-vintern))
    vc = vgates * vc0 + vgates * vcellIn
    vh = vgates * numpy.tanh(vc)
    assert Y.shape == (1, 1, 1) and C.shape == (1, 1, 1) and d.shape == (1, 1)
    assert_allclose(Y[0, 0, 0], vh, rtol=1e-6)
    assert_allclose(C[0, 0, 0], vc, rtol=1e-6)
    assert_allclose(d[0, 0], vc, rtol=1e-6)


def test_generic_base_reference_zero_run():
    """tests/test_TFNativeOp.py:234-250 (test_NativeLstmCell_run): zero inputs and zero state give zero output."""
    n_time, n_batch, n_hidden = 2, 1, 3
    Y, H, d = oracle.lstm_generic_base_fwd(numpy.zeros((n_time, n_batch, 4 * n_hidden)), numpy.zeros((n_hidden, 4 * n_hidden)),
                                           numpy.zeros((n_batch, n_hidden)), numpy.ones((n_time, n_batch)))  # fmt: skip
    assert Y.shape == (n_time, n_batch, n_hidden) and numpy.abs(Y).max() == 0 and numpy.abs(d).max() == 0
    assert_allclose(H[:, :, n_hidden:], 0.5)  # sigmoid(0) in the three gate blocks
    assert numpy.abs(H[:, :, :n_hidden]).max() == 0  # cell state


@pytest.mark.parametrize("T,B,n", [(1, 1, 1), (7, 3, 4), (12, 5, 6)])
def test_generic_base_vs_loop(T, B, n):
    r = _random(T + n, T, B, n)
    Y, H, d = oracle.lstm_generic_base_fwd(r["Z"], r["V"], r["c0"], r["mask"], dtype=numpy.float64)
    Y2, C2, G2, cT = _loop(r["Z"], r["V"], numpy.zeros((B, n)), r["c0"], r["mask"], range(T))
    assert_allclose(Y, Y2, rtol=1e-12, atol=1e-14)
    assert_allclose(H, G2, rtol=1e-12, atol=1e-14)
    assert_allclose(d, cT, rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize("start,step", [(0, 1), (0, -1), (2, 1), (1, -2), (0, 3), (2, -1), (4, -3)])
def test_low_mem_vs_loop(start, step):
    """With a negative step the op runs from frame T-start-1 down to frame `start` (returnn/native_op.py:827-833; NativeLstm2
    runs down to frame 0)."""
    T, B, n, n_in = 9, 4, 5, 3
    r = _random(start * 3 + step + 20, T, B, n, n_in)
    Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, dtype=numpy.float64)
    frames = range(start, T, step) if step > 0 else range(T - start - 1, start - 1, step)
    assert len(frames) > 0
    Xp = r["X"] @ r["W"][:n_in] + r["b"]
    Y2, C2, _, cT = _loop(Xp, r["W"][n_in:], r["y0"], r["c0"], r["mask"], frames)
    assert_allclose(Y, Y2, rtol=1e-12, atol=1e-14)
    assert_allclose(C, C2, rtol=1e-12, atol=1e-14)
    assert_allclose(d, cT, rtol=1e-12, atol=1e-14)


def test_low_mem_no_frame_visited_is_refused():
    """2*start > T-1 with a negative step: the reference's loop body never runs and d is read from an unwritten C."""
    r = _random(1, 5, 2, 3, 2)
    with pytest.raises(ValueError):
        oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 3, -1)
    oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 2, -1)  # exactly frame 2


def test_siblings_vs_torch_lstm_full_length():
    T, B, n, n_in = 8, 3, 5, 4
    r = _random(5, T, B, n, n_in)
    ones = numpy.ones((T, B))
    Yt, hT, cT = torch_lstm(r["Z"], r["V"], numpy.zeros((B, n)), r["c0"])
    Y, H, d = oracle.lstm_generic_base_fwd(r["Z"], r["V"], r["c0"], ones, dtype=numpy.float64)
    assert_allclose(Y, Yt, rtol=1e-9, atol=1e-12)
    assert_allclose(d, cT, rtol=1e-9, atol=1e-12)
    Xp = r["X"] @ r["W"][:n_in] + r["b"]
    Yt, hT, cT = torch_lstm(Xp, r["W"][n_in:], r["y0"], r["c0"])
    Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], ones, 0, 1, dtype=numpy.float64)
    assert_allclose(Y, Yt, rtol=1e-9, atol=1e-12)
    assert_allclose(d, cT, rtol=1e-9, atol=1e-12)
    assert_allclose(Y[-1], hT, rtol=1e-9, atol=1e-12)


def test_siblings_agree_with_native_lstm2_where_semantics_coincide():
    """Right-padded masks, forward direction: valid frames never see a masked predecessor, so all three ops agree."""
    T, B, n, n_in = 10, 4, 6, 3
    r = _random(8, T, B, n, n_in)
    lens = numpy.array([10, 4, 7, 1])
    mask = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float64)
    Xp = r["X"] @ r["W"][:n_in] + r["b"]
    Y2, C2, H2, d2, _ = oracle.native_lstm2_fwd(Xp, r["W"][n_in:], r["y0"], r["c0"], mask, 0, 1, dtype=numpy.float64)
    Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], mask, 0, 1, dtype=numpy.float64)
    assert_allclose(Y, Y2, rtol=1e-12, atol=1e-14)
    assert_allclose(C, C2, rtol=1e-12, atol=1e-14)
    assert_allclose(d, d2, rtol=1e-12, atol=1e-14)
    Y3, C3, H3, d3, _ = oracle.native_lstm2_fwd(r["Z"], r["V"], numpy.zeros((B, n)), r["c0"], mask, 0, 1, dtype=numpy.float64)
    Yg, Hg, dg = oracle.lstm_generic_base_fwd(r["Z"], r["V"], r["c0"], mask, dtype=numpy.float64)
    assert_allclose(Yg, Y3, rtol=1e-12, atol=1e-14)
    assert_allclose(dg, d3, rtol=1e-12, atol=1e-14)
    assert_allclose(Hg[:, :, :n], C3, rtol=1e-12, atol=1e-14)
    valid = mask[:, :, None] > 0
    assert_allclose((Hg[:, :, n:] * valid), (H3[:, :, n:] * valid), rtol=1e-12, atol=1e-14)


def test_siblings_float32_and_errors():
    r = _random(3, 6, 3, 4, 2)
    a = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 0, 1, dtype=numpy.float32)
    b = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 0, 1, dtype=numpy.float64)
    for x, y in zip(a, b):
        assert x.dtype == numpy.float32
        assert_allclose(x, y, rtol=1e-4, atol=1e-5)
    with pytest.raises(ValueError):
        oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 6, 1)
    with pytest.raises(ValueError):
        oracle.lstm_generic_base_fwd(numpy.zeros((0, 3, 16)), r["V"], r["c0"], numpy.zeros((0, 3)))
    Y, C, d = oracle.lstm_low_mem_fwd(numpy.zeros((0, 3, 2)), r["W"], r["b"], r["y0"], r["c0"], numpy.zeros((0, 3)), 0, 1)
    assert_allclose(d, r["c0"], rtol=1e-6)


def _generic_base_loss(Z, V, c0, mask, GY, Gd):
    Y, H, d = oracle.lstm_generic_base_fwd(Z, V, c0, mask, dtype=numpy.float64)
    return float((Y * GY).sum() + (d * Gd).sum())


def test_generic_base_gradient_vs_finite_differences():
    """Central differences of the (pinned) forward oracle, all three inputs, holes in the mask."""
    T, B, n = 6, 3, 4
    r = _random(41, T, B, n)
    rng = numpy.random.default_rng(42)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    Y, H, d = oracle.lstm_generic_base_fwd(r["Z"], r["V"], r["c0"], r["mask"], dtype=numpy.float64)
    GY_dirty = GY + 2.0 * (1.0 - r["mask"])[:, :, None]  # error signals on masked frames must not matter
    DZ, DV, Dc = oracle.lstm_generic_base_bwd(r["V"], r["c0"], r["mask"], Y, H, GY_dirty, Gd, dtype=numpy.float64)
    got = {"Z": DZ, "V": DV, "c0": Dc}
    eps = 1e-6
    for name in ("Z", "V", "c0"):
        flat = r[name].reshape(-1)
        for idx in rng.choice(flat.size, size=min(flat.size, 70), replace=False):
            old = flat[idx]
            flat[idx] = old + eps
            lp = _generic_base_loss(r["Z"], r["V"], r["c0"], r["mask"], GY, Gd)
            flat[idx] = old - eps
            lm = _generic_base_loss(r["Z"], r["V"], r["c0"], r["mask"], GY, Gd)
            flat[idx] = old
            num = (lp - lm) / (2 * eps)
            assert abs(num - got[name].reshape(-1)[idx]) <= 2e-6 * max(1.0, abs(num)), (name, idx, num, got[name].reshape(-1)[idx])
    assert numpy.abs(DZ * (1.0 - r["mask"])[:, :, None]).max() == 0.0  # masked frames get no gradient


def test_generic_base_gradient_vs_torch_autograd():
    """Autograd through a plain torch restatement of the forward pass (output of the frame before as recurrent input)."""
    import torch

    T, B, n = 7, 4, 5
    r = _random(43, T, B, n)
    rng = numpy.random.default_rng(44)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    Z = torch.tensor(r["Z"], requires_grad=True)
    V = torch.tensor(r["V"], requires_grad=True)
    c = torch.tensor(r["c0"], requires_grad=True)
    mask = torch.tensor(r["mask"])
    y_prev, c_prev, ys = torch.zeros((B, n), dtype=torch.float64), c, []
    for t in range(T):
        z = Z[t] + y_prev @ V
        g, i, f, o = torch.tanh(z[:, :n]), torch.sigmoid(z[:, n : 2 * n]), torch.sigmoid(z[:, 2 * n : 3 * n]), torch.sigmoid(z[:, 3 * n :])
        m = mask[t][:, None]
        c_new = (c_prev * f + g * i) * m + c_prev * (1 - m)
        y_prev, c_prev = torch.tanh(c_new) * o * m, c_new
        ys.append(y_prev)
    ((torch.stack(ys) * torch.tensor(GY)).sum() + (c_prev * torch.tensor(Gd)).sum()).backward()
    Y, H, d = oracle.lstm_generic_base_fwd(r["Z"], r["V"], r["c0"], r["mask"], dtype=numpy.float64)
    DZ, DV, Dc = oracle.lstm_generic_base_bwd(r["V"], r["c0"], r["mask"], Y, H, GY, Gd, dtype=numpy.float64)
    assert_allclose(DZ, Z.grad.numpy(), rtol=1e-8, atol=1e-10)
    assert_allclose(DV, V.grad.numpy(), rtol=1e-8, atol=1e-10)
    assert_allclose(Dc, c.grad.numpy(), rtol=1e-8, atol=1e-10)


def test_generic_base_gradient_float32_close_to_float64():
    T, B, n = 12, 3, 6
    r = _random(45, T, B, n)
    rng = numpy.random.default_rng(46)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    out = {}
    for dt in (numpy.float32, numpy.float64):
        Y, H, d = oracle.lstm_generic_base_fwd(r["Z"], r["V"], r["c0"], r["mask"], dtype=dt)
        out[dt] = oracle.lstm_generic_base_bwd(r["V"], r["c0"], r["mask"], Y, H, GY, Gd, dtype=dt)
    for a, b in zip(out[numpy.float32], out[numpy.float64]):
        assert numpy.abs(a - b).max() <= 2e-5 * max(1.0, numpy.abs(b).max())


def _low_mem_loss(r, start, step, GY, Gd):
    Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, dtype=numpy.float64)
    return float((Y * GY).sum() + (d * Gd).sum())


LOW_MEM_GRAD_CASES = [
    # T, start, step, mask: frames the forward pass visits = frames the reference's gradient loop visits
    (6, 0, 1, "full"), (6, 0, -1, "full"), (7, 0, 2, "full"), (8, 1, 2, "full"), (7, 1, -1, "full"), (9, 2, -2, "full"),
    (6, 0, 1, "right-padded"), (9, 2, 3, "right-padded"),
]  # fmt: skip


def _low_mem_mask(kind, T, B, rng):
    if kind == "full":
        return numpy.ones((T, B))
    lens = rng.integers(1, T + 1, size=B)
    lens[0] = T
    return (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float64)


@pytest.mark.parametrize("T,start,step,kind", LOW_MEM_GRAD_CASES)
def test_low_mem_gradient_vs_finite_differences(T, start, step, kind):
    """Central differences of the (pinned) forward oracle for all five differentiable inputs."""
    B, n, n_in = 3, 4, 5
    r = _random(61 + T, T, B, n, n_in=n_in)
    rng = numpy.random.default_rng(62)
    r["mask"] = _low_mem_mask(kind, T, B, rng)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, dtype=numpy.float64)
    GY_dirty = GY + 3.0 * (1.0 - r["mask"])[:, :, None]  # error signals on masked frames must not matter
    DX, DW, Db, Dh, Dc = oracle.lstm_low_mem_bwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, Y, C, GY_dirty, Gd)
    got = {"X": DX, "W": DW, "b": Db, "y0": Dh, "c0": Dc}
    eps = 1e-6
    for name in ("X", "W", "b", "y0", "c0"):
        flat = r[name].reshape(-1)
        for idx in rng.choice(flat.size, size=min(flat.size, 50), replace=False):
            old = flat[idx]
            flat[idx] = old + eps
            lp = _low_mem_loss(r, start, step, GY, Gd)
            flat[idx] = old - eps
            lm = _low_mem_loss(r, start, step, GY, Gd)
            flat[idx] = old
            num = (lp - lm) / (2 * eps)
            assert abs(num - got[name].reshape(-1)[idx]) <= 3e-6 * max(1.0, abs(num)), (name, idx, num, got[name].reshape(-1)[idx])


def test_low_mem_gradient_vs_torch_autograd():
    """Autograd through a plain torch restatement of the forward pass, right-padded batch, both inputs of the stacked
    weight matrix."""
    import torch

    T, B, n, n_in = 8, 4, 5, 3
    r = _random(63, T, B, n, n_in=n_in)
    rng = numpy.random.default_rng(64)
    r["mask"] = _low_mem_mask("right-padded", T, B, rng)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    X, W, b, y0, c0 = (torch.tensor(r[k], requires_grad=True) for k in ("X", "W", "b", "y0", "c0"))
    mask = torch.tensor(r["mask"])
    y_prev, c_prev, ys = y0, c0, []
    for t in range(T):
        z = torch.cat([X[t], y_prev], dim=1) @ W + b
        g, i, f, o = torch.tanh(z[:, :n]), torch.sigmoid(z[:, n : 2 * n]), torch.sigmoid(z[:, 2 * n : 3 * n]), torch.sigmoid(z[:, 3 * n :])
        m = mask[t][:, None]
        c_new = (c_prev * f + g * i) * m + c_prev * (1 - m)
        y_prev, c_prev = torch.tanh(c_new) * o * m, c_new
        ys.append(y_prev)
    ((torch.stack(ys) * torch.tensor(GY)).sum() + (c_prev * torch.tensor(Gd)).sum()).backward()
    Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 0, 1, dtype=numpy.float64)
    got = oracle.lstm_low_mem_bwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], 0, 1, Y, C, GY, Gd)
    for name, a, t in zip(("DX", "DW", "Db", "Dh", "Dc"), got, (X, W, b, y0, c0)):
        assert_allclose(a, t.grad.numpy(), rtol=1e-8, atol=1e-10, err_msg=name)


def test_low_mem_gradient_agrees_with_native_lstm2_gradient_on_full_batches():
    """With a full mask LstmLowMem is NativeLstm2 behind an input projection: DX = DXp W_x^T, DW = [X^T DXp; DW_rec],
    Db = column sums of DXp, where DXp and DW_rec come from the (separately pinned) NativeLstm2 gradient oracle."""
    T, B, n, n_in = 7, 3, 4, 6
    r = _random(65, T, B, n, n_in=n_in)
    r["mask"] = numpy.ones((T, B))
    rng = numpy.random.default_rng(66)
    GY, Gd = rng.normal(0, 1, (T, B, n)), rng.normal(0, 1, (B, n))
    for start, step in ((0, 1), (0, -1)):
        Y, C, d = oracle.lstm_low_mem_fwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, dtype=numpy.float64)
        DX, DW, Db, Dh, Dc = oracle.lstm_low_mem_bwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, Y, C, GY, Gd)
        Xp = r["X"] @ r["W"][:n_in] + r["b"]
        Y2, C2, H2, d2 = oracle.native_lstm2_fwd(Xp, r["W"][n_in:], r["y0"], r["c0"], r["mask"], start, step, dtype=numpy.float64)[:4]
        assert_allclose(Y2, Y, rtol=1e-12, atol=1e-12)
        DXp, DWr, Dy0, Dc0 = oracle.native_lstm2_bwd(Xp, r["W"][n_in:], r["y0"], r["c0"], r["mask"], start, step, Y2, C2, H2, GY, Gd, dtype=numpy.float64)
        assert_allclose(DX, DXp @ r["W"][:n_in].T, rtol=1e-9, atol=1e-11)
        assert_allclose(DW[:n_in], numpy.einsum("tbi,tbj->ij", r["X"], DXp), rtol=1e-9, atol=1e-11)
        assert_allclose(DW[n_in:], DWr, rtol=1e-9, atol=1e-11)
        assert_allclose(Db, DXp.sum(axis=(0, 1)), rtol=1e-9, atol=1e-11)
        assert_allclose(Dh, Dy0, rtol=1e-9, atol=1e-11)
        assert_allclose(Dc, Dc0, rtol=1e-9, atol=1e-11)


def test_low_mem_gradient_refuses_frame_sets_the_forward_pass_does_not_visit():
    T, B, n, n_in = 8, 2, 3, 2
    r = _random(67, T, B, n, n_in=n_in)
    z = numpy.zeros
    for start, step in ((0, 2), (2, 3), (1, -4)):  # T-1-start (or T-1-2*start) is not a multiple of the stride
        with pytest.raises(ValueError, match="stride"):
            oracle.lstm_low_mem_bwd(r["X"], r["W"], r["b"], r["y0"], r["c0"], r["mask"], start, step, z((T, B, n)), z((T, B, n)), z((T, B, n)), z((B, n)))
