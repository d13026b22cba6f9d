"""
``torch.nn.LSTM`` on the CPU as the library routine the LSTM layer is checked against, driven the way the
reference's torch backend drives ``torch.lstm`` (returnn/torch/frontend/_backend.py:2765-2850): frontend
parameters used as they are (``[4n,in]``, ``[4n,n]``, gate order input, forget, cell-in, output), the bias split
half and half over PyTorch's two bias vectors, ragged batches packed by their lengths, padded frames zero.
"""

from __future__ import annotations

import numpy
import torch


def blstm_layer(x, lens, fwd, bwd, h0=None, c0=None, dtype=torch.float64):
    """
    One bidirectional layer.

    :param x: [T,B,in] numpy
    :param lens: [B] or None
    :param fwd, bwd: {"ff_weight" [4n,in], "rec_weight" [4n,n], "bias" [4n] or None}
    :param h0, c0: [2,B,n] (forward, backward) or None for zeros
    :return: out [T,B,2n] (forward | backward), h [2,B,n], c [2,B,n] as float64 numpy
    """
    x = torch.as_tensor(numpy.asarray(x), dtype=dtype)
    T, B, d_in = x.shape
    n = fwd["rec_weight"].shape[1]
    m = torch.nn.LSTM(d_in, n, num_layers=1, bias=True, bidirectional=True).to(dtype)
    with torch.no_grad():
        for suffix, p in (("", fwd), ("_reverse", bwd)):
            getattr(m, "weight_ih_l0" + suffix).copy_(torch.as_tensor(numpy.asarray(p["ff_weight"]), dtype=dtype))
            getattr(m, "weight_hh_l0" + suffix).copy_(torch.as_tensor(numpy.asarray(p["rec_weight"]), dtype=dtype))
            b = p.get("bias")
            b = torch.zeros(4 * n, dtype=dtype) if b is None else torch.as_tensor(numpy.asarray(b), dtype=dtype)
            getattr(m, "bias_ih_l0" + suffix).copy_(b * 0.5)
            getattr(m, "bias_hh_l0" + suffix).copy_(b * 0.5)
        h0 = torch.zeros(2, B, n, dtype=dtype) if h0 is None else torch.as_tensor(numpy.asarray(h0), dtype=dtype)
        c0 = torch.zeros(2, B, n, dtype=dtype) if c0 is None else torch.as_tensor(numpy.asarray(c0), dtype=dtype)
        if lens is None:
            out, (h, c) = m(x, (h0, c0))
        else:
            packed = torch.nn.utils.rnn.pack_padded_sequence(
                x, torch.as_tensor(numpy.asarray(lens), dtype=torch.int64), enforce_sorted=False
            )
            out, (h, c) = m(packed, (h0, c0))
            out, _ = torch.nn.utils.rnn.pad_packed_sequence(out, total_length=T)
    return out.double().numpy(), h.double().numpy(), c.double().numpy()
