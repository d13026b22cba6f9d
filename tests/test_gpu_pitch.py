"""
Arrays with a row pitch (``ldX``, ``ldY`` of ``rtn_lstm2_call``; ``ldY``, ``ldDY``, ``ldDX`` of ``rtn_lstm2_bwd_call``): the
two directions of a bidirectional layer reading their gates from ONE projection [T,B,8n], writing ONE output [T,B,2n],
and in the gradient reading the error of that output and writing the error of that projection -- against the same calls
on contiguous copies (bit for bit: the pitch only moves addresses), and against the oracle.
"""

from __future__ import annotations

import numpy
import pytest
import torch

from oracle import lstm2_oracle as oracle
from returnn_amd import lib, torch_native_op
from returnn_amd import lstm as rlstm

from _gpu_util import announce, get_op, random_problem, to_dev

pytestmark = pytest.mark.gpu

POISON = 12345.0  # what the columns between the rows hold; the library must not touch them


def _pair_problem(seed, T, B, n):
    X, W, y0, c0, i = random_problem(seed, T, B, n)
    Xb, Wb, y0b, c0b, _ = random_problem(seed + 1, T, B, n)
    return [(X, W, y0, c0, i), (Xb, Wb, y0b, c0b, i)]


def _fwd_multi(problems, steps, dtype, mode, *, gap_x, gap_y, pitched):
    """
    Both problems through ``rtn_native_lstm2_fwd_multi``.  pitched: X of problem k is columns [k*(4n+gap_x), +4n) of one
    array and Y columns [k*(n+gap_y), +n) of one array; else every array on its own, contiguous.
    :return: per problem (Y, C, H, d) as tensors, and the joint Y array (or None)
    """
    get_op()
    cabi = lib.load()
    T, B = problems[0][4].shape
    n = problems[0][2].shape[1]
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    md = lib.MODES[mode]
    ldX, ldY = 2 * (4 * n + gap_x), 2 * (n + gap_y)
    Xj = torch.full((T, B, ldX), POISON, dtype=act, device="cuda:0")
    Yj = torch.full((T, B, ldY), POISON, dtype=act, device="cuda:0")
    arr = (lib.Lstm2Call * 2)()
    keep, outs = [], []
    for k, (X, W, y0, c0, i) in enumerate(problems):
        Wd, y0d = to_dev(W, dtype), to_dev(y0, dtype)
        c0d, id_ = to_dev(c0, "f32"), to_dev(i, "f32")
        if pitched:
            Xd = Xj[:, :, k * (4 * n + gap_x) : k * (4 * n + gap_x) + 4 * n]
            Xd.copy_(to_dev(X, dtype))
            Y = Yj[:, :, k * (n + gap_y) : k * (n + gap_y) + n]
        else:
            Xd = to_dev(X, dtype)
            Y = torch.full((T, B, n), float("nan"), dtype=act, device="cuda:0")
        C = torch.full((T, B, n), float("nan"), dtype=torch.float32, device="cuda:0")
        H = torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0")
        d = torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda:0")
        keep.append((Xd, Wd, y0d, c0d, id_))
        outs.append((Y, C, H, d))
        arr[k] = lib.Lstm2Call(Xd.data_ptr(), Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), 0, steps[k],
                               Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr(),
                               ldX if pitched else 0, ldY if pitched else 0)  # fmt: skip
    nbytes = int(cabi.rtn_native_lstm2_fwd_multi_workspace_bytes(2, T, B, n, dt, md))
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    lib.check(cabi.rtn_native_lstm2_fwd_multi(arr, 2, T, B, n, dt, md, ws.data_ptr(), ws.numel(), stream))
    lib.check(cabi.rtn_native_lstm2_fwd_multi_status(ws.data_ptr(), 2, T, B, n, dt, md, stream))
    torch.cuda.synchronize()
    return outs, keep, (Yj if pitched else None)


@pytest.mark.parametrize(
    "dtype,mode,T,B,n,gap_x,gap_y",
    [
        ("bf16", "auto", 12, 32, 1024, 0, 0),     # the benchmark's layer: [T,B,8n] in, [T,B,2n] out
        ("bf16", "auto", 9, 32, 1024, 64, 8),     # the same with unused columns between the directions
        ("bf16", "auto", 7, 13, 256, 0, 0),       # a last group of fewer rows
        ("f32", "auto", 8, 16, 512, 0, 0),
        ("f32", "auto", 6, 9, 64, 12, 4),
        ("f32", "stepwise", 5, 4, 96, 0, 0),      # one launch per frame
        ("f32", "graph", 5, 4, 96, 8, 4),
        ("f32", "auto", 5, 3, 24, 0, 0),          # element-wise kernels (widths below 32)
        ("f32", "auto", 6, 4, 100, 0, 0),         # runs zero-padded: the pitch is that of the caller's arrays
        ("bf16", "auto", 5, 8, 200, 8, 8),
        ("bf16", "auto", 6, 1, 512, 0, 0),        # a single sequence
    ],
)
def test_forward_of_both_directions_in_place(dtype, mode, T, B, n, gap_x, gap_y):
    announce("pitched forward", dtype, mode, T, B, n, gap_x, gap_y)
    problems = _pair_problem(300 + T + n, T, B, n)
    steps = (1, -1)
    got, keep, Yj = _fwd_multi(problems, steps, dtype, mode, gap_x=gap_x, gap_y=gap_y, pitched=True)
    want, _, _ = _fwd_multi(problems, steps, dtype, mode, gap_x=0, gap_y=0, pitched=False)
    f = lambda t: t.float().cpu().numpy()  # noqa: E731
    for k in range(2):
        for name, a, b in zip("YCHd", got[k], want[k]):
            assert numpy.isfinite(f(a)).all(), (k, name)
            assert numpy.array_equal(f(a), f(b)), "direction %i: %s differs from the contiguous call" % (k, name)
        # the pitched X was what the contiguous call read; last outputs come from pitched Y as well
        Xd, Wd, y0d, c0d, id_ = keep[k]
        last = torch_native_op.lstm_last_output(got[k][0], y0d, id_, 0, steps[k])
        last_c = torch_native_op.lstm_last_output(want[k][0], y0d, id_, 0, steps[k])
        assert torch.equal(last, last_c)
        X, W, y0, c0, i = problems[k]
        g = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
        Yo, Co, Ho, do = oracle.native_lstm2_fwd(g(Xd), g(Wd), g(y0d), c0, i, 0, steps[k], dtype=numpy.float64)[:4]
        tol = 2e-2 if dtype == "bf16" else 2e-5
        assert float(numpy.abs(f(got[k][0]) - Yo).max()) <= tol
        assert float(numpy.abs(f(got[k][3]) - do).max()) <= tol * 4
    if gap_y:
        gaps = torch.cat([Yj[:, :, n : n + gap_y], Yj[:, :, 2 * n + gap_y :]], dim=-1)
        assert bool((gaps == POISON).all()), "columns between the rows of Y were written"


@pytest.mark.parametrize(
    "dtype,T,B,n,gap",
    [
        ("bf16", 10, 32, 1024, 0),   # the benchmark's layer: one cooperative launch for both directions
        ("bf16", 8, 16, 256, 8),
        ("f32", 9, 20, 64, 0),
        ("f32", 6, 9, 128, 4),
        ("f32", 6, 5, 20, 0),        # element-wise gradient kernels
        ("f32", 6, 9, 100, 0),       # zero-padded run
        ("bf16", 5, 12, 200, 8),
    ],
)
@pytest.mark.parametrize("strided", [False, True])
def test_gradient_of_both_directions_in_place(dtype, T, B, n, gap, strided):
    """Y and DY as columns of [T,B,2n(+gaps)] arrays, DX into one [T,B,8n(+gaps)] array, against contiguous arrays."""
    announce("pitched gradient", dtype, T, B, n, gap, strided)
    problems = _pair_problem(500 + T + n, T, B, n)
    # (strided: steps +2 / -2, which leaves frames unvisited -- their DX rows must be cleared, the gaps left alone)
    starts, steps = ((1, 0), (2, -2)) if strided else ((0, 0), (1, -1))
    get_op()
    cabi = lib.load()
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    op = get_op()
    ldY, ldDX = 2 * (n + gap), 2 * (4 * n + 4 * gap)
    Yj = torch.full((T, B, ldY), POISON, dtype=act, device="cuda:0")
    DYj = torch.full((T, B, ldY), POISON, dtype=act, device="cuda:0")
    DXj = torch.full((T, B, ldDX), POISON, dtype=act, device="cuda:0")
    results = {}
    for pitched in (True, False):
        arr = (lib.Lstm2BwdCall * 2)()
        keep, outs = [], []
        for k, (X, W, y0, c0, i) in enumerate(problems):
            Xd, Wd, y0d = (to_dev(a, dtype) for a in (X, W, y0))
            c0d, id_ = to_dev(c0, "f32"), to_dev(i, "f32")
            Y, C, H, _ = op(Xd, Wd, y0d, c0d, id_, starts[k], steps[k])
            DY = to_dev(numpy.random.default_rng(40 + k).normal(0, 1.0, (T, B, n)).astype(numpy.float32), dtype)
            Dd = to_dev(numpy.random.default_rng(50 + k).normal(0, 1.0, (B, n)).astype(numpy.float32), "f32")
            if pitched:
                Yv, DYv = (J[:, :, k * (n + gap) : k * (n + gap) + n] for J in (Yj, DYj))
                Yv.copy_(Y)
                DYv.copy_(DY)
                DX = DXj[:, :, k * 4 * (n + gap) : k * 4 * (n + gap) + 4 * n]
            else:
                Yv, DYv = Y, DY
                DX = torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0")
            DW = torch.full((n, 4 * n), float("nan"), dtype=torch.float32, device="cuda:0")
            Dy0 = torch.full((B, n), float("nan"), dtype=act, device="cuda:0")
            Dc0 = torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda:0")
            keep.append((Xd, Wd, y0d, c0d, id_, Y, C, H, DY, Dd, Yv, DYv))
            outs.append((DX, DW, Dy0, Dc0))
            arr[k] = lib.Lstm2BwdCall(
                Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), starts[k], steps[k], Yv.data_ptr(), C.data_ptr(),
                H.data_ptr(), DYv.data_ptr(), Dd.data_ptr(), DX.data_ptr(), DW.data_ptr(), Dy0.data_ptr(), Dc0.data_ptr(),
                ldY if pitched else 0, ldY if pitched else 0, ldDX if pitched else 0,
            )  # fmt: skip
        nbytes = int(cabi.rtn_native_lstm2_bwd_multi_workspace_bytes(2, T, B, n, dt))
        ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device="cuda:0")
        stream = torch.cuda.current_stream().cuda_stream
        lib.check(cabi.rtn_native_lstm2_bwd_multi(arr, 2, T, B, n, dt, ws.data_ptr(), ws.numel(), stream))
        torch.cuda.synchronize()
        results[pitched] = (outs, keep)
    f = lambda t: t.float().cpu().numpy()  # noqa: E731
    g = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    tol = 2e-2 if dtype == "bf16" else 2e-5
    for k in range(2):
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), results[True][0][k], results[False][0][k]):
            assert numpy.isfinite(f(a)).all(), (k, name)
            assert numpy.array_equal(f(a), f(b)), "direction %i: %s differs from the contiguous call" % (k, name)
        Xd, Wd, y0d, c0d, id_, Y, C, H, DY, Dd, _, _ = results[True][1][k]
        X, W, y0, c0, i = problems[k]
        want = oracle.native_lstm2_bwd(g(Xd), g(Wd), g(y0d), c0, i, starts[k], steps[k], g(Y), g(C), g(H), g(DY), g(Dd), dtype=numpy.float64)
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), results[True][0][k], want):
            scale = max(float(numpy.abs(b).max()), 1e-30)
            assert float(numpy.abs(g(a) - b).max()) / scale <= tol, (k, name)
    if gap:
        gaps = torch.cat([DXj[:, :, 4 * n : 4 * (n + gap)], DXj[:, :, 4 * (n + gap) + 4 * n :]], dim=-1)
        assert bool((gaps == POISON).all()), "columns between the rows of DX were written"


def test_pitch_errors():
    announce("pitch errors")
    get_op()
    cabi = lib.load()
    T, B, n = 3, 2, 32
    z = torch.zeros((T * B * 8 * n,), dtype=torch.float32, device="cuda:0").data_ptr()
    ws = torch.empty((lib.workspace_bytes(T, B, n, lib.DTYPE_F32, lib.MODE_AUTO),), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream

    def call(ldX, ldY):
        arr = (lib.Lstm2Call * 1)()
        arr[0] = lib.Lstm2Call(z, z, z, z, z, 0, 1, z, z, z, z, ldX, ldY)
        return cabi.rtn_native_lstm2_fwd_multi(arr, 1, T, B, n, lib.DTYPE_F32, lib.MODE_AUTO, ws.data_ptr(), ws.numel(), stream)

    assert call(4 * n - 4, 0) == lib.RTN_ERR_ARG and "below the row length" in lib.last_error()
    assert call(0, n - 4) == lib.RTN_ERR_ARG and "below the row length" in lib.last_error()
    assert call(4 * n + 2, 0) == lib.RTN_ERR_ARG and "16-byte aligned" in lib.last_error()
    assert call(0, n + 1) == lib.RTN_ERR_ARG and "16-byte aligned" in lib.last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,T,B,n_in,n", [("bf16", 9, 8, 64, 256), ("f32", 7, 5, 40, 64), ("f32", 6, 3, 20, 24)])
def test_blstm_on_one_projection_equals_two_layers(dtype, T, B, n_in, n):
    """``blstm`` (one projection, outputs in place, gradient the same way) against two ``lstm`` calls and a concat."""
    announce("blstm one projection", dtype, T, B, n_in, n)
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    gen = torch.Generator().manual_seed(5)
    params = []
    for _ in range(2):
        params.append(tuple(
            (torch.randn(shape, generator=gen) * 0.2).to("cuda:0").requires_grad_(True)
            for shape in ((4 * n, n_in), (4 * n, n), (4 * n,))
        ))  # fmt: skip
    x = torch.randn((T, B, n_in), generator=gen).to("cuda:0").to(act)
    h0 = [(torch.randn((B, n), generator=gen) * 0.3).to("cuda:0").to(act) for _ in range(2)]
    c0 = [(torch.randn((B, n), generator=gen) * 0.3).to("cuda:0") for _ in range(2)]
    lens = torch.tensor([T] + [max(1, T - 1 - (b % 4)) for b in range(1, B)])
    G = torch.randn((T, B, 2 * n), generator=gen).to("cuda:0")

    def loss_of(y, sf, sb):
        return (y.float() * G).sum() + sf.h.float().sum() + 0.5 * sb.h.float().sum() + sf.c.sum() - sb.c.sum()

    def grads():
        out = [p.grad.clone() for ps in params for p in ps]
        for ps in params:
            for p in ps:
                p.grad = None
        return out

    w = rlstm.prepare_blstm_weights(params[0], params[1], dtype=act)
    y, sf, sb = rlstm.blstm(x, weights=w, state_fwd=rlstm.LstmState(h0[0], c0[0]), state_bwd=rlstm.LstmState(h0[1], c0[1]), seq_lens=lens)
    assert y.is_contiguous() and tuple(y.shape) == (T, B, 2 * n)
    loss_of(y, sf, sb).backward()
    got = grads()
    ys, states = [], []
    for k, direction in enumerate((1, -1)):
        yk, (hk, ck) = rlstm.lstm(x, state_h=h0[k], state_c=c0[k], ff_weight=params[k][0], rec_weight=params[k][1], bias=params[k][2],
                                  seq_lens=lens, direction=direction)  # fmt: skip
        ys.append(yk)
        states.append(rlstm.LstmState(hk, ck))
    y2 = torch.cat(ys, dim=-1)
    loss_of(y2, *states).backward()
    want = grads()
    torch.cuda.synchronize()
    # the recurrences see the same projected values (the one GEMM over [in,8n] gives each column what the two GEMMs over
    # [in,4n] give it, up to the GEMM library's choice of kernel per shape)
    tol = 2e-2 if dtype == "bf16" else 1e-4
    assert float((y.detach().float() - y2.detach().float()).abs().max()) <= tol
    for a, b in zip((sf.h, sf.c, sb.h, sb.c), (states[0].h, states[0].c, states[1].h, states[1].c)):
        assert float((a.detach().float() - b.detach().float()).abs().max()) <= tol * 2
    for a, b in zip(got, want):
        scale = max(float(b.abs().max()), 1e-30)
        assert float((a - b).abs().max()) / scale <= (4e-2 if dtype == "bf16" else 2e-4)
    # without gradients: the same outputs, through the multi-call entry with a joint output
    with torch.no_grad():
        y3, sf3, sb3 = rlstm.blstm(x, weights=w, state_fwd=rlstm.LstmState(h0[0], c0[0]), state_bwd=rlstm.LstmState(h0[1], c0[1]), seq_lens=lens)
    assert torch.equal(y3, y.detach()) and torch.equal(sf3.c, sf.c.detach()) and torch.equal(sb3.h, sb.h.detach())


def test_blstm_module_keeps_the_ops_layout_and_trains_like_two_lstm_modules():
    """:class:`BLSTM` (parameters in the op's layout, nothing converted per step) against two :class:`LSTM` modules
    holding the same weights: outputs, states and every parameter's gradient."""
    announce("BLSTM module")
    T, B, n_in, n = 8, 6, 48, 64
    gen = torch.Generator().manual_seed(11)
    singles = [rlstm.LSTM(n_in, n, device="cuda:0") for _ in range(2)]
    with torch.no_grad():
        for m in singles:
            for p in m.parameters():
                p.copy_((torch.randn(p.shape, generator=gen) * 0.2).to("cuda:0"))
    layer = rlstm.BLSTM(n_in, n, device="cuda:0")
    layer.load_frontend_params(*[m.frontend_params() for m in singles])
    x = torch.randn((T, B, n_in), generator=gen).to("cuda:0")
    lens = torch.tensor([T, T - 1, 3, T, 1, 5])
    G = torch.randn((T, B, 2 * n), generator=gen).to("cuda:0")
    y, sf, sb = layer(x, seq_lens=lens)
    ((y * G).sum() + sf.c.sum() + 2.0 * sb.h.sum()).backward()
    s0 = singles[0].default_initial_state(batch_dims=(B,))
    outs = [m(x, state=s0, seq_lens=lens, direction=d) for m, d in zip(singles, (1, -1))]
    y2 = torch.cat([o[0] for o in outs], dim=-1)
    ((y2 * G).sum() + outs[0][1].c.sum() + 2.0 * outs[1][1].h.sum()).backward()
    torch.cuda.synchronize()
    assert float((y.detach() - y2.detach()).abs().max()) <= 1e-5
    assert float((sb.h.detach() - outs[1][1].h.detach()).abs().max()) <= 1e-5

    def close(got, want, what):
        scale = max(float(want.abs().max()), 1e-30)
        assert float((got - want).abs().max()) / scale <= 1e-4, what

    n4 = 4 * n
    for k, (m, rec) in enumerate(zip(singles, (layer.rec_fwd, layer.rec_bwd))):
        close(layer.ff.grad[k * n4 : (k + 1) * n4], m.ff.grad, "ff %i" % k)
        close(rec.grad, m.rec.grad, "rec %i" % k)
        close(layer.bias.grad[k * n4 : (k + 1) * n4], m.bias.grad, "bias %i" % k)
    # a checkpoint written by the layer is in the frontend's layout
    sd = layer.state_dict()
    assert torch.equal(sd["bwd.rec_weight"], singles[1].state_dict()["rec_weight"])
    assert torch.equal(sd["fwd.ff_weight"], singles[0].state_dict()["ff_weight"])
