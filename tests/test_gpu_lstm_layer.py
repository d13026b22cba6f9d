"""
GPU parity of the LSTM layer (projection GEMM + NativeLstm2 through the C ABI + final state) and of the
bidirectional encoder stack against ``torch.nn.LSTM`` on the CPU in float64, packed by the sequence lengths --
what the reference's frontend test asserts for ``rf.LSTM`` (tests/test_rf_rec.py:13-74) and how its torch backend
computes it (returnn/torch/frontend/_backend.py:2765-2850).

Tolerances: float32 1e-5 relative (+2e-6 absolute floor for values near zero); bfloat16 weights and activations
2e-2 absolute on outputs and states of one layer fed identical inputs.
"""

from __future__ import annotations

import numpy
import pytest
import torch
from numpy.testing import assert_allclose

from returnn_amd import lstm as rlstm
from returnn_amd import synthetic
from _gpu_util import announce, get_op
from _torch_ref import blstm_layer

pytestmark = pytest.mark.gpu

F32_RTOL, F32_ATOL = 1e-5, 2e-6
BF16_ATOL = 2e-2
DEV = "cuda:0"


def _params(rng, n, d_in, bias=True):
    return {
        "ff_weight": synthetic.glorot_uniform(rng, (4 * n, d_in)),
        "rec_weight": synthetic.glorot_uniform(rng, (4 * n, n)),
        "bias": rng.standard_normal(4 * n).astype(numpy.float32) * 0.3 if bias else None,
    }


def _dev(a, dtype=torch.float32):
    return None if a is None else torch.from_numpy(numpy.asarray(a, dtype=numpy.float32)).to(DEV).to(dtype)


def _np(t):
    return t.detach().float().cpu().numpy().astype(numpy.float64)


@pytest.mark.parametrize("ragged", [False, True])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("T,B,d_in,n", [(9, 5, 7, 13), (40, 16, 24, 64), (33, 7, 80, 128), (12, 6, 20, 100)])
def test_lstm_f32_vs_torch(T, B, d_in, n, ragged, bias):
    announce("lstm layer f32", T, B, d_in, n, ragged, bias)
    get_op()
    rng = numpy.random.default_rng(T * 131 + n)
    x = rng.standard_normal((T, B, d_in)).astype(numpy.float32)
    lens = rng.integers(1, T + 1, size=(B,)) if ragged else None
    if ragged:
        lens[0] = T
    fwd, bwd = _params(rng, n, d_in, bias), _params(rng, n, d_in, bias)
    h0 = rng.standard_normal((2, B, n)).astype(numpy.float32) * 0.5
    c0 = rng.standard_normal((2, B, n)).astype(numpy.float32) * 0.5
    out, h, c = blstm_layer(x, lens, fwd, bwd, h0, c0)
    for k, (p, direction) in enumerate(((fwd, 1), (bwd, -1))):
        y, (hn, cn) = rlstm.lstm(
            _dev(x), state_h=_dev(h0[k]), state_c=_dev(c0[k]), ff_weight=_dev(p["ff_weight"]),
            rec_weight=_dev(p["rec_weight"]), bias=_dev(p["bias"]),
            seq_lens=None if lens is None else torch.from_numpy(lens), direction=direction,
        )  # fmt: skip
        assert y.shape == (T, B, n) and y.dtype == torch.float32
        assert_allclose(_np(y), out[:, :, k * n : (k + 1) * n], rtol=F32_RTOL, atol=F32_ATOL)
        assert_allclose(_np(hn), h[k], rtol=F32_RTOL, atol=F32_ATOL)
        assert_allclose(_np(cn), c[k], rtol=F32_RTOL, atol=F32_ATOL)


def test_lstm_single_step_and_chaining():
    """A single step equals T=1 (tests/test_rf_rec.py:46-74), and stepping frame by frame with the returned state
    equals one call over the whole sequence."""
    announce("lstm layer single step")
    get_op()
    rng = numpy.random.default_rng(5)
    T, B, d_in, n = 6, 4, 7, 13
    x = rng.standard_normal((T, B, d_in)).astype(numpy.float32)
    p = _params(rng, n, d_in)
    m = rlstm.LSTM(d_in, n, device=DEV)
    m.load_frontend_params({k: _dev(p[k]) for k in ("ff_weight", "rec_weight", "bias")})
    h0 = (rng.standard_normal((B, n)) * 0.5).astype(numpy.float32)
    c0 = (rng.standard_normal((B, n)) * 0.5).astype(numpy.float32)
    s = rlstm.LstmState(h=_dev(h0), c=_dev(c0))
    y_all, s_all = m(_dev(x), state=s)
    ys = []
    for t in range(T):
        y, s = m(_dev(x[t]), state=s)
        assert y.shape == (B, n)
        assert torch.equal(y, s.h)
        ys.append(y)
    assert_allclose(_np(torch.stack(ys)), _np(y_all), rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(_np(s.h), _np(s_all.h), rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(_np(s.c), _np(s_all.c), rtol=F32_RTOL, atol=F32_ATOL)
    out, h, c = blstm_layer(x, None, p, p, numpy.stack([h0, h0]), numpy.stack([c0, c0]))
    assert_allclose(_np(y_all), out[:, :, :n], rtol=F32_RTOL, atol=F32_ATOL)
    assert_allclose(_np(s_all.c), c[0], rtol=F32_RTOL, atol=F32_ATOL)


def test_module_follows_parameter_updates():
    announce("lstm layer parameter update")
    get_op()
    m = rlstm.LSTM(8, 16, device=DEV)
    s = m.default_initial_state(batch_dims=(3,))
    x = torch.randn(5, 3, 8, device=DEV)
    y1, _ = m(x, state=s)
    y1b, _ = m(x, state=s)
    assert torch.equal(y1, y1b)
    with torch.no_grad():
        m.rec.mul_(0.5)
    y2, _ = m(x, state=s)
    fp = m.frontend_params()
    ref, _ = rlstm.lstm(x, state_h=s.h, state_c=s.c, ff_weight=fp["ff_weight"], rec_weight=fp["rec_weight"], bias=fp["bias"])
    assert torch.equal(y2, ref) and not torch.equal(y1, y2)


@pytest.mark.parametrize("T,B,d_in,n", [(50, 32, 80, 256), (30, 16, 512, 256)])
def test_lstm_bf16_vs_torch(T, B, d_in, n):
    """bf16 weights and activations, one layer, both directions, against float64 on the same float32 parameters."""
    announce("lstm layer bf16", T, B, d_in, n)
    get_op()
    rng = numpy.random.default_rng(n + T)
    x = rng.standard_normal((T, B, d_in)).astype(numpy.float32)
    lens = rng.integers(T // 2, T + 1, size=(B,))
    lens[0] = T
    fwd, bwd = _params(rng, n, d_in), _params(rng, n, d_in)
    out, h, c = blstm_layer(x, lens, fwd, bwd)
    bf = torch.bfloat16
    for k, (p, direction) in enumerate(((fwd, 1), (bwd, -1))):
        y, (hn, cn) = rlstm.lstm(
            _dev(x, bf), state_h=torch.zeros(B, n, dtype=bf, device=DEV), state_c=torch.zeros(B, n, device=DEV),
            ff_weight=_dev(p["ff_weight"], bf), rec_weight=_dev(p["rec_weight"], bf), bias=_dev(p["bias"], bf),
            seq_lens=torch.from_numpy(lens), direction=direction,
        )  # fmt: skip
        assert y.dtype == bf and hn.dtype == bf and cn.dtype == torch.float32
        assert_allclose(_np(y), out[:, :, k * n : (k + 1) * n], rtol=0, atol=BF16_ATOL)
        assert_allclose(_np(hn), h[k], rtol=0, atol=BF16_ATOL)
        assert_allclose(_np(cn), c[k], rtol=0, atol=BF16_ATOL)


def _reference_stack(prob, dtype=torch.float32):
    """Per-layer outputs of the stack with torch.nn.LSTM on the CPU."""
    x = prob.features
    outs, states = [], []
    for layer in prob.layers:
        out, h, c = blstm_layer(x, prob.lens, layer["fwd"], layer["bwd"], dtype=dtype)
        outs.append(out)
        states.append((h, c))
        x = out
    return outs, states


def test_blstm_encoder_f32_vs_torch():
    announce("blstm encoder f32")
    get_op()
    prob = synthetic.make_encoder_config("cfg4", T=40, B=8, n=64, num_layers=3, bias_std=0.2)
    outs, states = _reference_stack(prob, torch.float64)
    enc = rlstm.BlstmEncoder.from_params(prob.layers, device=DEV)
    y, st = enc(_dev(prob.features), seq_lens=torch.from_numpy(prob.lens), collect_states=True)
    assert y.shape == (40, 8, 128)
    assert_allclose(_np(y), outs[-1], rtol=3 * F32_RTOL, atol=3 * F32_ATOL)  # three layers deep
    for (sf, sb), (h, c) in zip(st, states):
        assert_allclose(_np(sf.h), h[0], rtol=3 * F32_RTOL, atol=3 * F32_ATOL)
        assert_allclose(_np(sb.h), h[1], rtol=3 * F32_RTOL, atol=3 * F32_ATOL)
        assert_allclose(_np(sf.c), c[0], rtol=3 * F32_RTOL, atol=3 * F32_ATOL)
        assert_allclose(_np(sb.c), c[1], rtol=3 * F32_RTOL, atol=3 * F32_ATOL)
    pad = numpy.arange(40)[:, None] >= prob.lens[None, :]
    assert float(numpy.abs(_np(y)[pad]).max(initial=0.0)) == 0.0


def test_blstm_encoder_cfg4_reduced_bf16():
    """
    The 6-layer encoder at its real widths (80 -> 2048 -> ... , n=1024 per direction, B=32) on a shortened batch.
    Each layer is checked on its own against float32 torch on the CPU fed the same input (the previous layer's GPU
    output), to the 2e-2 bound of a single bf16 layer; the end-to-end deviation through all six layers is printed
    and held to a looser bound, since bf16 rounding of the activations compounds from layer to layer.
    """
    announce("blstm encoder cfg4 reduced bf16")
    get_op()
    prob = synthetic.make_encoder_config("cfg4", T=48)
    bf = torch.bfloat16
    enc = rlstm.BlstmEncoder.from_params(prob.layers, device=DEV, dtype=bf)
    lens = torch.from_numpy(prob.lens)
    x = _dev(prob.features, bf)
    x_ref_chain = prob.features
    B = prob.B
    worst_layer, worst_chain = 0.0, 0.0
    for li in range(prob.num_layers):
        layer = prob.layers[li]
        s0 = rlstm.LstmState(h=torch.zeros(B, prob.n, dtype=bf, device=DEV), c=torch.zeros(B, prob.n, device=DEV))
        outs = []
        for d, direction in (("fwd", 1), ("bwd", -1)):  # the two directions as single layers, from the frontend's parameters
            yd, (hd, cd) = rlstm.lstm(x, state_h=s0.h, state_c=s0.c, seq_lens=lens, direction=direction,
                                      **{k: _dev(layer[d][k], bf) for k in ("ff_weight", "rec_weight", "bias")})  # fmt: skip
            outs.append((yd, rlstm.LstmState(hd, cd)))
        (yf, sf), (yb, sb) = outs
        y = torch.cat((yf, yb), dim=-1)
        ref, h, c = blstm_layer(_np(x), prob.lens, layer["fwd"], layer["bwd"], dtype=torch.float32)
        err = float(numpy.abs(_np(y) - ref).max())
        err_c = max(float(numpy.abs(_np(sf.c) - c[0]).max()), float(numpy.abs(_np(sb.c) - c[1]).max()))
        worst_layer = max(worst_layer, err, err_c)
        chain, _, _ = blstm_layer(x_ref_chain, prob.lens, layer["fwd"], layer["bwd"], dtype=torch.float32)
        worst_chain = max(worst_chain, float(numpy.abs(_np(y) - chain).max()))
        print("layer %i: max |y - ref(same input)| = %.4g, |c| %.4g, end-to-end %.4g" % (li, err, err_c, worst_chain), flush=True)
        x_ref_chain = chain
        x = y
    full = enc(_dev(prob.features, bf), seq_lens=lens)
    assert torch.equal(full, x)
    assert worst_layer <= BF16_ATOL
    assert worst_chain <= 5e-2


@pytest.mark.parametrize("n", [32, 40])
def test_blstm_layer_gradients_vs_torch(n):
    """Training through the layer: gradients of all parameters, the input and the initial states equal those of a
    bidirectional torch.nn.LSTM on the CPU in float64 (loss on the outputs and on both final states).  n=40 is a width
    that the ops run zero-padded."""
    announce("blstm layer gradients", n)
    get_op()
    rng = numpy.random.default_rng(21)
    T, B, d_in = 11, 6, 10
    x = rng.standard_normal((T, B, d_in)).astype(numpy.float32)
    lens = numpy.array([11, 3, 7, 1, 11, 5])
    fwd, bwd = _params(rng, n, d_in), _params(rng, n, d_in)
    h0 = (rng.standard_normal((2, B, n)) * 0.5).astype(numpy.float32)
    c0 = (rng.standard_normal((2, B, n)) * 0.5).astype(numpy.float32)
    G = rng.standard_normal((T, B, 2 * n)).astype(numpy.float32)
    Gh = rng.standard_normal((2, B, n)).astype(numpy.float32)
    Gc = rng.standard_normal((2, B, n)).astype(numpy.float32)

    # reference: torch.nn.LSTM, float64, CPU
    dt = torch.float64
    m = torch.nn.LSTM(d_in, n, bidirectional=True).to(dt)
    with torch.no_grad():
        for sfx, p in (("", fwd), ("_reverse", bwd)):
            getattr(m, "weight_ih_l0" + sfx).copy_(torch.as_tensor(p["ff_weight"], dtype=dt))
            getattr(m, "weight_hh_l0" + sfx).copy_(torch.as_tensor(p["rec_weight"], dtype=dt))
            getattr(m, "bias_ih_l0" + sfx).copy_(torch.as_tensor(p["bias"], dtype=dt) * 0.5)
            getattr(m, "bias_hh_l0" + sfx).copy_(torch.as_tensor(p["bias"], dtype=dt) * 0.5)
    xr = torch.tensor(x, dtype=dt, requires_grad=True)
    h0r = torch.tensor(h0, dtype=dt, requires_grad=True)
    c0r = torch.tensor(c0, dtype=dt, requires_grad=True)
    packed = torch.nn.utils.rnn.pack_padded_sequence(xr, torch.as_tensor(lens), enforce_sorted=False)
    out, (hT, cT) = m(packed, (h0r, c0r))
    out, _ = torch.nn.utils.rnn.pad_packed_sequence(out, total_length=T)
    ((out * torch.tensor(G, dtype=dt)).sum() + (hT * torch.tensor(Gh, dtype=dt)).sum() + (cT * torch.tensor(Gc, dtype=dt)).sum()).backward()

    # this package, float32, GPU
    mods = []
    for p in (fwd, bwd):
        mod = rlstm.LSTM(d_in, n, device=DEV)
        mod.load_frontend_params({k: _dev(p[k]) for k in ("ff_weight", "rec_weight", "bias")})
        mods.append(mod)
    xg = _dev(x).requires_grad_(True)
    h0g = _dev(h0).requires_grad_(True)
    c0g = _dev(c0).requires_grad_(True)
    y, sf, sb = rlstm.blstm(xg, fwd=mods[0].weights(torch.float32), bwd=mods[1].weights(torch.float32),
                            state_fwd=rlstm.LstmState(h0g[0], c0g[0]), state_bwd=rlstm.LstmState(h0g[1], c0g[1]),
                            seq_lens=torch.from_numpy(lens))  # fmt: skip
    loss = (y * _dev(G)).sum() + (sf.h * _dev(Gh[0])).sum() + (sb.h * _dev(Gh[1])).sum() + (sf.c * _dev(Gc[0])).sum() + (sb.c * _dev(Gc[1])).sum()
    loss.backward()
    assert_allclose(_np(y), out.detach().numpy(), rtol=F32_RTOL, atol=F32_ATOL)

    def close(got, want, what):
        want = want.detach().numpy() if isinstance(want, torch.Tensor) else want
        scale = max(float(numpy.abs(want).max()), 1e-30)
        assert float(numpy.abs(_np(got) - want).max()) / scale <= 3e-5, what

    close(xg.grad, xr.grad, "x")
    close(h0g.grad, h0r.grad, "h0")
    close(c0g.grad, c0r.grad, "c0")
    for mod, sfx in zip(mods, ("", "_reverse")):
        # (the module's parameters are in the op's layout: back to torch's gate order and orientation)
        close(rlstm._from_native_gate_order(mod.ff.grad), getattr(m, "weight_ih_l0" + sfx).grad, "ff_weight" + sfx)
        close(rlstm._from_native_gate_order(mod.rec.grad.t()), getattr(m, "weight_hh_l0" + sfx).grad, "rec_weight" + sfx)
        close(rlstm._from_native_gate_order(mod.bias.grad), getattr(m, "bias_ih_l0" + sfx).grad, "bias" + sfx)  # either half of torch's bias sees the gradient of the sum


def test_lstm_module_trains_one_step():
    """The module under an optimizer: one SGD step lowers a simple loss (forward and gradient op end to end, bf16)."""
    announce("lstm module trains")
    get_op()
    torch.manual_seed(0)
    mod = rlstm.LSTM(16, 32, device=DEV, dtype=torch.bfloat16)
    x = torch.randn(20, 8, 16, device=DEV).bfloat16()
    target = torch.randn(20, 8, 32, device=DEV) * 0.1
    lens = torch.tensor([20, 20, 15, 9, 20, 3, 12, 20])
    s0 = mod.default_initial_state(batch_dims=(8,))
    opt = torch.optim.SGD(mod.parameters(), lr=0.5)
    losses = []
    for _ in range(3):
        opt.zero_grad()
        y, _ = mod(x, state=s0, seq_lens=lens)
        loss = ((y.float() - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(numpy.isfinite(losses)) and losses[-1] < losses[0], losses


def test_lstm_module_training_step_recorded_into_a_graph():
    """Forward, loss and backward of the module under stream capture (the reference engine captures whole training steps,
    returnn/torch/util/graph_capture.py): after eager warm-up steps the graph is replayed with new inputs and must give
    the parameter and input gradients of the eager step (the recorded gradient op takes another decomposition than the
    eager one: equal up to bfloat16 rounding)."""
    announce("lstm module captured training step")
    get_op()
    torch.manual_seed(1)
    T, B, d_in, n = 14, 8, 16, 64
    mod = rlstm.LSTM(d_in, n, device=DEV, dtype=torch.bfloat16)
    x = torch.randn(T, B, d_in, device=DEV).bfloat16().requires_grad_(True)
    target = torch.randn(T, B, n, device=DEV) * 0.1
    lens = torch.tensor([14, 14, 9, 5, 14, 2, 11, 14], device=DEV)
    s0 = mod.default_initial_state(batch_dims=(B,))
    params = list(mod.parameters())

    def step():
        y, _ = mod(x, state=s0, seq_lens=lens)
        loss = ((y.float() - target) ** 2).mean()
        return torch.autograd.grad(loss, [x] + params)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        recorded = step()
    for k in range(3):
        with torch.no_grad():
            x.copy_(torch.randn(T, B, d_in, device=DEV).bfloat16())
            target.copy_(torch.randn(T, B, n, device=DEV) * 0.1)
        graph.replay()
        torch.cuda.synchronize()
        got = [g.clone() for g in recorded]
        eager = step()
        torch.cuda.synchronize()
        for idx, (a, e) in enumerate(zip(got, eager)):
            scale = max(float(e.float().abs().max()), 1e-30)
            assert float((a.float() - e.float()).abs().max()) / scale <= 2e-2, (k, idx)
