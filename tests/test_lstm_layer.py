"""
CPU checks of the LSTM layer's host logic: the parameter mapping onto the op (gate reorder, transpose,
projection outside the op, mask from lengths, direction) is pinned by running the mapped problem through the
CPU oracle and comparing with ``torch.nn.LSTM`` on the packed batch -- the behaviour the reference's frontend
test expects of the layer (tests/test_rf_rec.py:13-43 via the torch backend).
"""

from __future__ import annotations

import math

import numpy
import pytest
import torch
from numpy.testing import assert_allclose

from oracle import lstm2_oracle as oracle
from returnn_amd import lstm as rlstm
from returnn_amd import synthetic
from _torch_ref import blstm_layer


def _params(rng, n, d_in, bias=True):
    return {
        "ff_weight": synthetic.glorot_uniform(rng, (4 * n, d_in)),
        "rec_weight": synthetic.glorot_uniform(rng, (4 * n, n)),
        "bias": rng.standard_normal(4 * n).astype(numpy.float32) * 0.3 if bias else None,
    }


def _layer_via_oracle(x, lens, p, h0, c0, direction):
    """The steps of returnn_amd.lstm.lstm with numpy and the oracle in place of the GPU."""
    w = rlstm.prepare_weights(
        torch.from_numpy(p["ff_weight"]), torch.from_numpy(p["rec_weight"]),
        None if p["bias"] is None else torch.from_numpy(p["bias"]), dtype=torch.float32,
    )  # fmt: skip
    T, B, _ = x.shape
    X = x.astype(numpy.float64) @ w.ff.numpy().astype(numpy.float64)
    if w.bias is not None:
        X = X + w.bias.numpy()[None, None, :]
    mask = numpy.ones((T, B), numpy.float32) if lens is None else rlstm.sequence_mask_time_major(torch.as_tensor(lens), maxlen=T).numpy()
    Y, C, H, d, y_last = oracle.native_lstm2_fwd(X, w.rec.numpy(), h0, c0, mask, 0, direction, dtype=numpy.float64)
    return Y, y_last, d


@pytest.mark.parametrize("ragged", [False, True])
@pytest.mark.parametrize("bias", [False, True])
def test_mapping_matches_torch_lstm(ragged, bias):
    rng = numpy.random.default_rng(11)
    T, B, d_in, n = 9, 5, 7, 13  # dims of the reference's frontend test
    x = rng.standard_normal((T, B, d_in)).astype(numpy.float32)
    lens = numpy.array([9, 3, 1, 7, 9]) if ragged else None
    fwd, bwd = _params(rng, n, d_in, bias), _params(rng, n, d_in, bias)
    h0 = rng.standard_normal((2, B, n)).astype(numpy.float32) * 0.5
    c0 = rng.standard_normal((2, B, n)).astype(numpy.float32) * 0.5
    out, h, c = blstm_layer(x, lens, fwd, bwd, h0, c0)
    for k, (p, direction) in enumerate(((fwd, 1), (bwd, -1))):
        Y, y_last, d = _layer_via_oracle(x, lens, p, h0[k], c0[k], direction)
        assert_allclose(Y, out[:, :, k * n : (k + 1) * n], rtol=1e-9, atol=1e-12)
        assert_allclose(y_last, h[k], rtol=1e-9, atol=1e-12)
        assert_allclose(d, c[k], rtol=1e-9, atol=1e-12)


def test_gate_reorder_is_a_permutation_of_blocks():
    n = 3
    w = torch.arange(4 * n, dtype=torch.float32)[:, None] * torch.ones(1, 2)
    lw = rlstm.prepare_weights(w, torch.zeros(4 * n, n), torch.arange(4 * n, dtype=torch.float32))
    # input, forget, cell-in, output -> cell-in, input, forget, output
    expect = list(range(2 * n, 3 * n)) + list(range(0, n)) + list(range(n, 2 * n)) + list(range(3 * n, 4 * n))
    assert lw.ff.shape == (2, 4 * n) and lw.rec.shape == (n, 4 * n)
    assert lw.ff[0].tolist() == expect and lw.bias.tolist() == expect
    assert lw.ff.t().is_contiguous() and lw.rec.is_contiguous()  # (ff: a transposed view, see prepare_weights)


def test_sequence_mask_time_major():
    m = rlstm.sequence_mask_time_major(torch.tensor([3, 0, 5]), maxlen=5)
    assert m.dtype == torch.float32 and m.shape == (5, 3)
    assert m.t().tolist() == [[1, 1, 1, 0, 0], [0, 0, 0, 0, 0], [1, 1, 1, 1, 1]]


def test_module_parameters_and_init():
    torch.manual_seed(0)
    m = rlstm.LSTM(80, 64)
    # parameters in the op's layout; the frontend's layout and names in the state dict
    assert m.ff.shape == (256, 80) and m.rec.shape == (64, 256) and m.bias.shape == (256,)
    sd = m.state_dict()
    assert sorted(sd) == ["bias", "ff_weight", "rec_weight"]
    assert sd["ff_weight"].shape == (256, 80) and sd["rec_weight"].shape == (256, 64) and sd["bias"].shape == (256,)
    assert float(m.bias.detach().abs().max()) == 0.0
    for p in (sd["ff_weight"], sd["rec_weight"]):
        limit = math.sqrt(6.0 / sum(p.shape))
        assert float(p.abs().max()) <= limit
        assert float(p.abs().max()) > 0.9 * limit
        assert abs(float(p.var()) - limit * limit / 3.0) < 0.1 * limit * limit / 3.0  # variance 1/fan_avg
    assert rlstm.LSTM(4, 4, with_bias=False).bias is None
    s = m.default_initial_state(batch_dims=(3,))
    assert s.h.shape == (3, 64) and s.c.shape == (3, 64) and float(s.h.abs().sum() + s.c.abs().sum()) == 0.0


def test_module_state_dict_speaks_the_frontend_layout():
    """What the module keeps is the op's layout (gate blocks cell-in, input, forget, output; the recurrent matrix
    transposed); what it saves and loads is the frontend's (returnn/tf/frontend_layers/_backend.py:1199-1222)."""
    n, d_in = 3, 2
    m = rlstm.LSTM(d_in, n)
    ff = torch.arange(4 * n * d_in, dtype=torch.float32).reshape(4 * n, d_in)
    rec = 100.0 + torch.arange(4 * n * n, dtype=torch.float32).reshape(4 * n, n)
    bias = 1000.0 + torch.arange(4 * n, dtype=torch.float32)
    m.load_state_dict({"ff_weight": ff, "rec_weight": rec, "bias": bias})
    i, f, g, o = (slice(k * n, (k + 1) * n) for k in range(4))  # the frontend's blocks: input, forget, cell-in, output
    assert torch.equal(m.ff.detach(), torch.cat((ff[g], ff[i], ff[f], ff[o])))
    assert torch.equal(m.rec.detach(), torch.cat((rec[g], rec[i], rec[f], rec[o])).t())
    assert torch.equal(m.bias.detach(), torch.cat((bias[g], bias[i], bias[f], bias[o])))
    w = m.weights(torch.float32)
    ref = rlstm.prepare_weights(ff, rec, bias)
    assert torch.equal(w.ff, ref.ff) and torch.equal(w.rec, ref.rec) and torch.equal(w.bias, ref.bias)
    sd = m.state_dict()
    assert torch.equal(sd["ff_weight"], ff) and torch.equal(sd["rec_weight"], rec) and torch.equal(sd["bias"], bias)
    m2 = rlstm.LSTM(d_in, n)
    m2.load_state_dict(sd)
    assert all(torch.equal(a, b) for a, b in zip(m.parameters(), m2.parameters()))
    with pytest.raises(RuntimeError, match="ff_weight"):
        m2.load_state_dict({"ff_weight": ff[:, :1], "rec_weight": rec, "bias": bias})
    with pytest.raises(RuntimeError, match="Missing"):
        m2.load_state_dict({"ff_weight": ff, "bias": bias})


def test_no_cpu_implementation():
    m = rlstm.LSTM(4, 8)
    s = m.default_initial_state(batch_dims=(2,))
    with pytest.raises(RuntimeError, match="HIP"):
        m(torch.zeros(3, 2, 4), state=s)


def test_argument_errors():
    m = rlstm.LSTM(4, 8)
    s = m.default_initial_state(batch_dims=(2,))
    with pytest.raises(ValueError, match="in_dim"):
        m(torch.zeros(3, 2, 5), state=s)
    with pytest.raises(ValueError, match="needs attributes"):
        m(torch.zeros(3, 2, 4), state=rlstm.LstmState(h=None, c=s.c))
    with pytest.raises(ValueError, match="rec_weight"):
        rlstm.prepare_weights(torch.zeros(32, 4), torch.zeros(32, 9), None)
    with pytest.raises(ValueError, match="bias"):
        rlstm.prepare_weights(torch.zeros(32, 4), torch.zeros(32, 8), torch.zeros(31))


def test_encoder_config_shapes():
    p = synthetic.make_encoder_config("cfg4", T=20, B=3, n=16, num_layers=3)
    assert p.features.shape == (20, 3, 80) and p.lens.shape == (3,) and p.lens[0] == 20
    assert p.lens.min() >= 10 and p.lens.max() <= 20
    assert [l["fwd"]["ff_weight"].shape for l in p.layers] == [(64, 80), (64, 32), (64, 32)]
    assert all(l[k]["rec_weight"].shape == (64, 16) for l in p.layers for k in ("fwd", "bwd"))
    w = p.layers[1]["bwd"]["ff_weight"]
    assert numpy.abs(w).max() <= math.sqrt(6.0 / (64 + 32))
    enc = rlstm.BlstmEncoder.from_params(p.layers)
    assert enc.num_layers == 3 and enc.in_dim == 80 and enc.out_dim == 16
    # the layers keep their parameters in the op's layout and hand the frontend's back, bit for bit
    back = enc.layers[2].frontend_params()
    for d in ("fwd", "bwd"):
        for k in ("ff_weight", "rec_weight", "bias"):
            assert torch.equal(back[d][k], torch.from_numpy(p.layers[2][d][k])), (d, k)
    assert tuple(enc.layers[1].ff.shape) == (128, 32) and tuple(enc.layers[1].rec_bwd.shape) == (16, 64)
    sd = enc.state_dict()
    assert torch.equal(sd["layers.2.bwd.rec_weight"], torch.from_numpy(p.layers[2]["bwd"]["rec_weight"]))
    other = rlstm.BlstmEncoder(80, 16, 3)
    other.load_state_dict(sd)
    assert all(torch.equal(a, b) for a, b in zip(enc.parameters(), other.parameters()))
    # the op's layout is what prepare_blstm_weights makes of the frontend's parameters
    w = enc.layers[1].weights(torch.float32)
    w2 = rlstm.prepare_blstm_weights(
        *[tuple(torch.from_numpy(p.layers[1][d][k]) for k in ("ff_weight", "rec_weight", "bias")) for d in ("fwd", "bwd")]
    )
    assert all(torch.equal(a, b) for a, b in zip(w, w2))
    del sd["layers.0.fwd.bias"]
    with pytest.raises(RuntimeError, match="layers.0.fwd.bias"):
        other.load_state_dict(sd)
