"""
Independent references used to pin the oracle (and through it the HIP path).

``textbook_lstm`` follows the structure of the reference's own check, the unrolled textbook LSTM
in tests/test_TFNativeOp.py:467-608 (``lstm_step_op`` / ``pure_tf_unrolled_lstm``): it takes the
*unprojected* input x with W_f and b, blends state with the mask instead of zeroing the output,
and iterates over an explicit list of visited frames.  It shares no code with ``oracle/``.

``torch_lstm`` drives ``torch.nn.LSTM`` (gate order i,f,g,o and [4n,n] weights) with weights
converted from the op's layout ([n,4n], order cell-in,input,forget,output), packed for ragged
lengths the way the reference's torch backend does (returnn/torch/frontend/_backend.py:2796-2822).
"""

from __future__ import annotations

import numpy


def sigmoid(x):
    return 1.0 / (1.0 + numpy.exp(-x))


def textbook_lstm(x, h_0, c_0, mask, W_f, W_r, b, start=0, step=1, dtype=numpy.float64):
    """
    :param x: [T,B,n_in]
    :param h_0, c_0: [B,n]
    :param mask: [T,B]
    :param W_f: [n_in,4n]  W_r: [n,4n]  b: [4n]
    :return: h [T,B,n], c [T,B,n] (zeros on frames that are not visited), c_T, h_T
    """
    x, h_0, c_0, mask, W_f, W_r, b = (numpy.asarray(a, dtype=dtype) for a in (x, h_0, c_0, mask, W_f, W_r, b))
    n_time = x.shape[0]
    n = h_0.shape[1]
    assert n_time > 0 and 0 <= start < n_time and step != 0
    if step >= 0:
        visited = list(range(start, n_time, step))
    else:
        visited = list(range(n_time - start - 1, -1, step))
    h = numpy.zeros((n_time,) + h_0.shape, dtype=dtype)
    c = numpy.zeros((n_time,) + c_0.shape, dtype=dtype)
    h_t, c_t = h_0, c_0
    for t in visited:
        intern = x[t] @ W_f + h_t @ W_r + b[None, :]
        cell_in = numpy.tanh(intern[:, :n])
        inp_gate = sigmoid(intern[:, n : 2 * n])
        fgt_gate = sigmoid(intern[:, 2 * n : 3 * n])
        out_gate = sigmoid(intern[:, 3 * n :])
        c_new = c_t * fgt_gate + cell_in * inp_gate
        h_new = numpy.tanh(c_new) * out_gate
        m = mask[t][:, None]
        h_t = h_new * m + h_t * (1.0 - m)
        c_t = c_new * m + c_t * (1.0 - m)
        h[t] = h_t
        c[t] = c_t
    return h, c, c_t, h_t


def visited_slice(n_time, start, step):
    """The python slice of frames the op visits (tests/test_TFNativeOp.py:826-829, 851)."""
    start_ = start if step >= 0 else n_time - start - 1
    return slice(start_, None, step)


def reference_fixture(dtype=numpy.float32):
    """The deterministic inputs of the reference's ``lstm_kwargs`` (tests/test_TFNativeOp.py:866-889)."""
    n_time, n_batch, n_in, n = 3, 2, 1, 2
    mask = numpy.array([[1, 1, 0], [1, 0, 0]]).astype(dtype).transpose()

    def gen(shape, offset):
        return numpy.sin(numpy.arange(numpy.prod(shape)) + offset).reshape(shape).astype(dtype)

    return dict(
        x=gen((n_time, n_batch, n_in), 0.1),
        h_0=gen((n_batch, n), 0.2),
        c_0=gen((n_batch, n), 0.3),
        mask=mask,
        W_f=numpy.ones((n_in, 4 * n), dtype=dtype),
        W_r=numpy.ones((n, 4 * n), dtype=dtype),
        b=-numpy.ones((4 * n,), dtype=dtype),
    )


REFERENCE_START_STEP = [(0, 1), (0, -1), (1, 1), (1, -1), (0, 2), (0, -2)]  # tests/test_TFNativeOp.py:824


def torch_lstm(X, W, y0, c0, lens=None, reverse=False):
    """
    ``torch.nn.LSTM`` on the same problem, float64.  The op's X is already projected, so the
    input weight of torch's LSTM is the identity (in the op's gate order mapped to torch's).

    :param X: [T,B,4n] op layout (cell-in, input, forget, output)
    :param W: [n,4n]
    :param lens: optional [B] lengths (right padded); packed like the reference's torch backend
    :param reverse: process each sequence from its last valid frame to its first
    :return: Y [T,B,n] (zeros on padded frames), h_T [B,n], c_T [B,n]
    """
    import torch

    X = torch.as_tensor(numpy.asarray(X, dtype=numpy.float64))
    T, B, n4 = X.shape
    n = n4 // 4
    # op order: g(cell-in), i, f, o  ->  torch order: i, f, g, o
    perm = numpy.concatenate([numpy.arange(n, 2 * n), numpy.arange(2 * n, 3 * n), numpy.arange(0, n), numpy.arange(3 * n, 4 * n)])
    Wt = torch.as_tensor(numpy.asarray(W, dtype=numpy.float64))[:, perm].T.contiguous()  # [4n,n]
    Xt = X[:, :, perm]
    lstm = torch.nn.LSTM(input_size=4 * n, hidden_size=n, bias=False, bidirectional=reverse).double()
    with torch.no_grad():
        eye = torch.eye(4 * n, dtype=torch.float64)
        lstm.weight_ih_l0.copy_(eye)
        lstm.weight_hh_l0.copy_(Wt)
        if reverse:
            lstm.weight_ih_l0_reverse.copy_(eye)
            lstm.weight_hh_l0_reverse.copy_(Wt)
    h0 = torch.as_tensor(numpy.asarray(y0, dtype=numpy.float64))[None]
    c0_ = torch.as_tensor(numpy.asarray(c0, dtype=numpy.float64))[None]
    if reverse:
        h0 = h0.repeat(2, 1, 1)
        c0_ = c0_.repeat(2, 1, 1)
    with torch.no_grad():
        if lens is None:
            out, (hT, cT) = lstm(Xt, (h0, c0_))
        else:
            packed = torch.nn.utils.rnn.pack_padded_sequence(Xt, torch.as_tensor(lens, dtype=torch.int64), enforce_sorted=False)
            out, (hT, cT) = lstm(packed, (h0, c0_))
            out, _ = torch.nn.utils.rnn.pad_packed_sequence(out, total_length=T)
    if reverse:
        return out[:, :, n:].numpy(), hT[1].numpy(), cT[1].numpy()
    return out.numpy(), hT[0].numpy(), cT[0].numpy()


def torch_lstm_grads(X, W, y0, c0, lens, reverse, GY, Gd):
    """Gradients of sum(Y*GY) + sum(c_final*Gd) through torch.nn.LSTM, mapped back to the op's layout."""
    import torch

    T, B, n4 = X.shape
    n = n4 // 4
    # op order: g(cell-in), i, f, o  ->  torch order: i, f, g, o
    perm = numpy.concatenate([numpy.arange(n, 2 * n), numpy.arange(2 * n, 3 * n), numpy.arange(0, n), numpy.arange(3 * n, 4 * n)])
    inv = numpy.argsort(perm)
    Xt = torch.tensor(X[:, :, perm], dtype=torch.float64, requires_grad=True)
    lstm = torch.nn.LSTM(input_size=4 * n, hidden_size=n, bias=False, bidirectional=reverse).double()
    sfx = "_reverse" if reverse else ""
    with torch.no_grad():
        for s in ("", "_reverse") if reverse else ("",):
            getattr(lstm, "weight_ih_l0" + s).copy_(torch.eye(4 * n, dtype=torch.float64))
            getattr(lstm, "weight_hh_l0" + s).copy_(torch.tensor(W[:, perm].T.copy()))
    k = 2 if reverse else 1
    h0 = torch.tensor(numpy.stack([y0] * k), requires_grad=True)
    c0_ = torch.tensor(numpy.stack([c0] * k), requires_grad=True)
    packed = torch.nn.utils.rnn.pack_padded_sequence(Xt, torch.as_tensor(lens, dtype=torch.int64), enforce_sorted=False)
    out, (hT, cT) = lstm(packed, (h0, c0_))
    out, _ = torch.nn.utils.rnn.pad_packed_sequence(out, total_length=T)
    sel = slice(n, 2 * n) if reverse else slice(0, n)
    loss = (out[:, :, sel] * torch.tensor(GY)).sum() + (cT[k - 1] * torch.tensor(Gd)).sum()
    loss.backward()
    DX = Xt.grad.numpy()[:, :, inv]
    DW = getattr(lstm, "weight_hh_l0" + sfx).grad.numpy().T[:, inv]
    return DX, DW, h0.grad.numpy()[k - 1], c0_.grad.numpy()[k - 1]
