"""
Writes the golden vectors of this directory.  Run from the repository root: ``python tests/golden/make_golden.py``.

The expected values come from implementations that share no code with ``oracle/`` or the HIP library and need nothing
from the reference tree: the textbook LSTM of tests/_textbook.py in float64 on the inputs of the reference's own fixture
(``lstm_kwargs``, tests/test_TFNativeOp.py:866-889, for its six (start, step) pairs, :824), ``torch.nn.LSTM`` in float64
on a packed ragged batch (forward results and, through autograd, the gradients of a fixed weighted-sum loss), and the
closed form of the reference's one-cell LstmLowMem test (tests/test_TFNativeOp.py:264-297).  Everything is stored as
float64 in ``.npz`` files (no pickles).
"""

from __future__ import annotations

import os
import sys

import numpy

_here = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(_here))

from _textbook import REFERENCE_START_STEP, reference_fixture, textbook_lstm, torch_lstm, torch_lstm_grads  # noqa: E402


def reference_fixture_vectors():
    fx = reference_fixture(numpy.float64)
    out = {k: v for k, v in fx.items()}
    out["X"] = fx["x"] @ fx["W_f"] + fx["b"][None, None, :]  # what the op gets: the projected input
    for start, step in REFERENCE_START_STEP:
        h, c, c_T, h_T = textbook_lstm(start=start, step=step, **fx)
        tag = "s%i_%s%i" % (start, "p" if step > 0 else "m", abs(step))
        out["h_" + tag], out["c_" + tag], out["cT_" + tag], out["hT_" + tag] = h, c, c_T, h_T
    return out


def torch_ragged_vectors():
    rng = numpy.random.default_rng(20240607)
    T, B, n = 9, 5, 16
    X = rng.normal(0, 0.7, (T, B, 4 * n))
    W = rng.normal(0, 1.0, (n, 4 * n)) / numpy.sqrt(n)
    y0, c0 = rng.normal(0, 0.4, (B, n)), rng.normal(0, 0.4, (B, n))
    lens = numpy.array([9, 4, 1, 7, 9])
    GY, Gd = rng.normal(0, 1.0, (T, B, n)), rng.normal(0, 1.0, (B, n))
    out = dict(X=X, W=W, y0=y0, c0=c0, lens=lens.astype(numpy.float64), GY=GY, Gd=Gd)
    for reverse in (False, True):
        tag = "rev" if reverse else "fwd"
        Y, hT, cT = torch_lstm(X, W, y0, c0, lens=lens, reverse=reverse)
        DX, DW, Dy0, Dc0 = torch_lstm_grads(X, W, y0, c0, lens, reverse, GY, Gd)
        for name, a in (("Y", Y), ("hT", hT), ("cT", cT), ("DX", DX), ("DW", DW), ("Dy0", Dy0), ("Dc0", Dc0)):
            out["%s_%s" % (name, tag)] = numpy.asarray(a, dtype=numpy.float64)
    return out


def low_mem_closed_form():
    vX, vb, vy0, vc0 = 0.2, 0.3, 0.1, 0.1
    vintern = vX + vy0 + vb
    vgates = 1.0 / (1.0 + numpy.exp(-vintern))
    vc = vgates * vc0 + vgates * numpy.tanh(vintern)
    return dict(X=numpy.full((1, 1, 1), vX), W=numpy.ones((2, 4)), b=numpy.full((4,), vb), y0=numpy.full((1, 1), vy0),
                c0=numpy.full((1, 1), vc0), Y=numpy.full((1, 1, 1), vgates * numpy.tanh(vc)), C=numpy.full((1, 1, 1), vc))  # fmt: skip


def main():
    for name, make in (("reference_fixture", reference_fixture_vectors), ("torch_ragged", torch_ragged_vectors), ("low_mem_closed_form", low_mem_closed_form)):
        path = os.path.join(_here, name + ".npz")
        numpy.savez(path, **{k: numpy.asarray(v, dtype=numpy.float64) for k, v in make().items()})
        print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
