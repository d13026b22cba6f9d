"""
GPU parity of the NativeLstm2 gradient op (C ABI ``rtn_native_lstm2_bwd``) against the CPU oracle of the reference's
gradient code, on the forward results of the HIP path itself.

Tolerances.  The north star fixes tolerances for the forward outputs only; gradients are sums over up to T*B terms
whose summation order differs between MFMA tiles and a sequential loop, so they are judged relative to the largest
magnitude of each array: float32 within 2e-5 of it (the float32 oracle itself is that far from the float64 oracle),
bfloat16 (bf16 activations, gates and DX; float32 accumulation) within 2e-2 of it.
"""

from __future__ import annotations

import numpy
import pytest
import torch

from oracle import lstm2_oracle as oracle
from returnn_amd import lib, synthetic, torch_native_op
from _gpu_util import announce, get_op, random_problem, to_dev

pytestmark = pytest.mark.gpu


def _rel_to_max(got, want):
    scale = max(float(numpy.abs(want).max()), 1e-30)
    return float(numpy.abs(got - want).max()) / scale


def _run(T, B, n, dtype, start, step, seed=0, scale_x=0.5):
    X, W, y0, c0, i = random_problem(seed, T, B, n, scale_x=scale_x)
    rng = numpy.random.default_rng(seed + 1000)
    DY = rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32)
    Dd = rng.normal(0, 1.0, (B, n)).astype(numpy.float32)
    op = get_op()
    Xd, Wd, y0d, DYd = (to_dev(a, dtype) for a in (X, W, y0, DY))
    c0d, id_, Ddd = (to_dev(a, "f32") for a in (c0, i, Dd))
    Y, C, H, d = op(Xd, Wd, y0d, c0d, id_, start, step)
    got = torch_native_op.native_lstm2_grad(Wd, y0d, c0d, id_, start, step, Y, C, H, DYd, Ddd)
    torch.cuda.synchronize()
    got = [g.float().cpu().numpy() for g in got]
    # the checker gets what the GPU's gradient op got: the GPU's own forward results and the same (rounded) inputs
    f = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    want = oracle.native_lstm2_bwd(f(Xd), f(Wd), f(y0d), c0, i, start, step, f(Y), f(C), f(H), f(DYd), Dd, dtype=numpy.float64)
    return got, want, (X, W, y0, c0, i, DY, Dd)


@pytest.mark.parametrize("start,step", [(0, 1), (0, -1), (1, 2), (2, -3)])
@pytest.mark.parametrize("T,B,n", [(7, 3, 16), (12, 20, 64), (9, 40, 128), (6, 5, 20), (5, 2, 3), (5, 9, 48), (4, 12, 400), (3, 9, 1024), (4, 20, 720)])
def test_bwd_f32(T, B, n, start, step):
    announce("bwd f32", T, B, n, start, step)
    got, want, _ = _run(T, B, n, "f32", start, step, seed=T + n)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert a.shape == b.shape
        assert _rel_to_max(a, b) <= 2e-5, (name, _rel_to_max(a, b))


@pytest.mark.parametrize("step", [1, -1])
@pytest.mark.parametrize("T,B,n", [(10, 16, 64), (16, 32, 256), (6, 5, 24), (6, 20, 768), (5, 33, 800), (5, 7, 48), (4, 24, 1280)])
def test_bwd_bf16(T, B, n, step):
    announce("bwd bf16", T, B, n, step)
    got, want, _ = _run(T, B, n, "bf16", 0, step, seed=T + n)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert _rel_to_max(a, b) <= 2e-2, (name, _rel_to_max(a, b))


# (rows per group, tiles per workgroup, wavefronts per workgroup): decompositions of the persistent gradient kernel that the
# plan picks for other shapes than the ones above -- one (row, k) pair per thread with 2 and 4 tiles, whole and half ring
# frames, 8 wavefronts -- forced here on a small problem with ragged sequence lengths and a last group of fewer rows.
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("rows,tiles,waves", [(8, 2, 4), (8, 4, 4), (4, 2, 4), (3, 4, 4), (16, 2, 4), (12, 1, 4), (8, 1, 8), (8, 2, 8), (8, 4, 8)])
def test_bwd_forced_decompositions(rows, tiles, waves, dtype):
    from _gpu_util import env

    T, B, n = 9, 21, 256
    announce("bwd forced decomposition", rows, tiles, waves, dtype)
    with env(RTN_LSTM2_BWD_KERNEL=2, RTN_LSTM2_BWD_ROWS=rows, RTN_LSTM2_BWD_MT=tiles, RTN_LSTM2_BWD_WAVES=waves):
        got, want, _ = _run(T, B, n, dtype, 1, 2 if tiles == 2 else -1, seed=rows + 10 * tiles + waves)
        plan = lib.bwd_plan_text()
    if "bwd_regw" not in plan:
        pytest.skip("no persistent kernel for this decomposition: " + plan)
    assert "rows_per_group=%i" % rows in plan and "tiles=%i" % tiles in plan and "waves=%i" % waves in plan, plan
    bar = 2e-2 if dtype == "bf16" else 2e-5
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert numpy.isfinite(a).all(), name
        assert _rel_to_max(a, b) <= bar, (name, _rel_to_max(a, b), plan)


def test_bwd_read_delay_only_moves_time():
    """The delay between a frame's stores and the read of its ring slot (and whether it adapts) decides how often a read is
    repeated, never what is read: every setting gives the same bits, on a plan with one pair per thread and on one without."""
    from _gpu_util import env

    announce("bwd read delay")
    for tiles in (2, 1):
        results = []
        for delay, inc in [(None, None), (0, 0), (64, 0), (3, 2)]:
            with env(RTN_LSTM2_BWD_KERNEL=2, RTN_LSTM2_BWD_ROWS=8, RTN_LSTM2_BWD_MT=tiles, RTN_LSTM2_BWD_POLL_DELAY=delay, RTN_LSTM2_BWD_DELAY_INC=inc):
                got, _, _ = _run(12, 19, 256, "bf16", 0, -1, seed=5)
                assert "bwd_regw" in lib.bwd_plan_text() and "tiles=%i" % tiles in lib.bwd_plan_text(), lib.bwd_plan_text()
            results.append(got)
        for other in results[1:]:
            for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), other, results[0]):
                assert numpy.array_equal(a, b), (tiles, name)


def test_bwd_groups_found_on_several_xcds_fall_back_to_device_scope():
    """With half the true XCD count the groups of an XCD-local gradient plan land on two XCDs each: the kernel's check
    finds that out and exchanges the ring at device scope (and adapts its read delay): the same bits, no abort."""
    from _gpu_util import env

    announce("bwd xcd-local with a wrong XCD count")
    T, B, n = 10, 32, 512
    want, _, _ = _run(T, B, n, "bf16", 0, 1, seed=3)
    plan = lib.bwd_plan_text()
    assert "bwd_regw_xcd" in plan, plan
    with env(RTN_LSTM2_XCDS=4):
        got, _, _ = _run(T, B, n, "bf16", 0, 1, seed=3)
        assert "bwd_regw_xcd" in lib.bwd_plan_text(), lib.bwd_plan_text()
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert numpy.isfinite(a).all(), name
        assert numpy.array_equal(a, b), name


def test_bwd_cfg2_reduced_f32():
    announce("bwd cfg2 reduced")
    p = synthetic.make_config("cfg2", T=60)
    rng = numpy.random.default_rng(2)
    DY = rng.normal(0, 1.0, (p.T, p.B, p.n)).astype(numpy.float32)
    Dd = rng.normal(0, 1.0, (p.B, p.n)).astype(numpy.float32)
    op = get_op()
    args = [to_dev(a, "f32") for a in (p.X, p.W, p.y0, p.c0, p.i)]
    Y, C, H, d = op(*args, 0, 1)
    got = torch_native_op.native_lstm2_grad(args[1], args[2], args[3], args[4], 0, 1, Y, C, H, to_dev(DY, "f32"), to_dev(Dd, "f32"))
    f = lambda t: t.float().cpu().numpy()  # noqa: E731
    want = oracle.native_lstm2_bwd(p.X, p.W, p.y0, p.c0, p.i, 0, 1, f(Y), f(C), f(H), DY, Dd, dtype=numpy.float64)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got, want):
        assert _rel_to_max(f(a), b) <= 2e-5, (name, _rel_to_max(f(a), b))


def test_bwd_autograd_function_matches_torch_lstm():
    """End to end through autograd: loss on Y and d, gradients equal those of torch.nn.LSTM on the CPU (float64)."""
    announce("bwd autograd")
    from test_oracle_bwd import torch_lstm_grads

    get_op()
    T, B, n = 9, 6, 32
    rng = numpy.random.default_rng(4)
    X = rng.normal(0, 0.7, (T, B, 4 * n)).astype(numpy.float32)
    W = (rng.normal(0, 1.0, (n, 4 * n)) / numpy.sqrt(n)).astype(numpy.float32)
    y0 = rng.normal(0, 0.4, (B, n)).astype(numpy.float32)
    c0 = rng.normal(0, 0.4, (B, n)).astype(numpy.float32)
    lens = numpy.array([9, 4, 1, 7, 9, 2])
    mask = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    GY = rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32)
    Gd = rng.normal(0, 1.0, (B, n)).astype(numpy.float32)
    for reverse in (False, True):
        want = torch_lstm_grads(*(a.astype(numpy.float64) for a in (X, W, y0, c0)), lens, reverse, GY.astype(numpy.float64), Gd.astype(numpy.float64))
        leaves = [to_dev(a, "f32").requires_grad_(True) for a in (X, W, y0, c0)]
        Y, C, H, d = torch_native_op.NativeLstm2Function.apply(*leaves, to_dev(mask, "f32"), 0, -1 if reverse else 1)
        assert not C.requires_grad and not H.requires_grad
        loss = (Y * to_dev(GY, "f32")).sum() + (d * to_dev(Gd, "f32")).sum()
        loss.backward()
        for name, leaf, b in zip(("X", "W", "y0", "c0"), leaves, want):
            assert _rel_to_max(leaf.grad.cpu().numpy().astype(numpy.float64), b) <= 2e-5, (name, reverse)


def test_bwd_edge_cases_and_errors():
    announce("bwd edge cases")
    get_op()
    cabi = lib.load()
    B, n = 3, 16
    z = lambda *s: torch.zeros(s, device="cuda:0")  # noqa: E731
    Dd = torch.ones((B, n), device="cuda:0")
    DX, DW, Dy0, Dc0 = torch_native_op.native_lstm2_grad(z(n, 4 * n), z(B, n), z(B, n), z(0, B), 0, 1, z(0, B, n), z(0, B, n),
                                                         z(0, B, 4 * n), z(0, B, n), Dd)  # fmt: skip
    assert DX.shape == (0, B, 4 * n) and float(DW.abs().max()) == 0 and float(Dy0.abs().max()) == 0 and bool((Dc0 == 1).all())
    with pytest.raises(RuntimeError, match="start"):
        torch_native_op.native_lstm2_grad(z(n, 4 * n), z(B, n), z(B, n), z(4, B), 9, 1, z(4, B, n), z(4, B, n), z(4, B, 4 * n), z(4, B, n), Dd)
    with pytest.raises(RuntimeError, match="shape"):
        torch_native_op.native_lstm2_grad(z(n, 4 * n), z(B, n), z(B, n), z(4, B), 0, 1, z(4, B, n), z(4, B, n), z(4, B, n), z(4, B, n), Dd)
    with pytest.raises(RuntimeError, match="HIP"):
        torch_native_op.native_lstm2_grad(*(t.cpu() for t in (z(n, 4 * n), z(B, n), z(B, n), z(4, B))), 0, 1,
                                          *(t.cpu() for t in (z(4, B, n), z(4, B, n), z(4, B, 4 * n), z(4, B, n), Dd)))  # fmt: skip
    assert cabi.rtn_native_lstm2_bwd_workspace_bytes(10, B, n, 0) > 0
    assert cabi.rtn_native_lstm2_bwd_workspace_bytes(-1, B, n, 0) == 0


@pytest.mark.parametrize("T,B,n,dtype", [(14, 32, 256, "bf16"), (9, 20, 64, "f32"), (20, 32, 1024, "bf16"), (6, 5, 20, "f32"), (7, 70, 128, "bf16"), (6, 9, 100, "f32"), (5, 12, 200, "bf16")])
def test_bwd_multi_equals_single_calls(T, B, n, dtype):
    """
    The two directions of a layer through ``rtn_native_lstm2_bwd_multi``: against the oracle to the same bar as a single
    call, and against two single calls.  The joint launch may use another decomposition (k tiles per workgroup), which
    changes the order in which the MFMA partial sums are added: equal to float32 rounding, i.e. within 1e-5 of the
    largest magnitude in float32 and within one bfloat16 step (2^-7) of it in bfloat16.
    """
    announce("bwd multi", T, B, n, dtype)
    X, W, y0, c0, i = random_problem(50 + T + n, T, B, n)
    Wb = numpy.ascontiguousarray(W[::-1])  # another matrix for the other direction
    rng = numpy.random.default_rng(77)
    DY = [rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32) for _ in range(2)]
    Dd = [rng.normal(0, 1.0, (B, n)).astype(numpy.float32) for _ in range(2)]
    op = get_op()
    Xd, y0d = to_dev(X, dtype), to_dev(y0, dtype)
    Wd = [to_dev(W, dtype), to_dev(Wb, dtype)]
    DYd = [to_dev(a, dtype) for a in DY]
    c0d, id_ = to_dev(c0, "f32"), to_dev(i, "f32")
    Ddd = [to_dev(a, "f32") for a in Dd]
    steps = (1, -1)
    fw = [op(Xd, Wd[k], y0d, c0d, id_, 0, steps[k]) for k in range(2)]
    calls = [(Wd[k], y0d, c0d, id_, 0, steps[k], fw[k][0], fw[k][1], fw[k][2], DYd[k], Ddd[k]) for k in range(2)]
    multi = torch_native_op.native_lstm2_grad_multi(calls)
    single = [torch_native_op.native_lstm2_grad(*c) for c in calls]
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    tol = 2e-5 if dtype == "f32" else 2e-2
    for k in range(2):
        Y, C, H, _ = fw[k]
        want = oracle.native_lstm2_bwd(f(Xd), f(Wd[k]), f(y0d), c0, i, 0, steps[k], f(Y), f(C), f(H), f(DYd[k]), Dd[k], dtype=numpy.float64)
        for name, a, s, b in zip(("DX", "DW", "Dy0", "Dc0"), multi[k], single[k], want):
            assert _rel_to_max(f(a), b) <= tol, (k, name, _rel_to_max(f(a), b))
            assert _rel_to_max(f(a), f(s)) <= (1e-5 if dtype == "f32" else 2.0**-7), (k, name, _rel_to_max(f(a), f(s)))


def test_bwd_multi_errors_and_empty():
    announce("bwd multi errors")
    get_op()
    cabi = lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    assert cabi.rtn_native_lstm2_bwd_multi(None, 0, 4, 2, 32, lib.DTYPE_F32, None, 0, stream) == 0  # nothing to do
    assert cabi.rtn_native_lstm2_bwd_multi(None, 2, 4, 2, 32, lib.DTYPE_F32, None, 0, stream) == lib.RTN_ERR_ARG
    assert cabi.rtn_native_lstm2_bwd_multi_workspace_bytes(2, 4, 2, 32, lib.DTYPE_F32) == 2 * cabi.rtn_native_lstm2_bwd_workspace_bytes(4, 2, 32, lib.DTYPE_F32)
    with pytest.raises(RuntimeError, match="one shape"):
        z = lambda *s: torch.zeros(*s, device="cuda:0")  # noqa: E731
        a = (z(8, 32), z(2, 8), z(2, 8), z(3, 2), 0, 1, z(3, 2, 8), z(3, 2, 8), z(3, 2, 32), z(3, 2, 8), z(2, 8))
        b = (z(8, 32), z(2, 8), z(2, 8), z(4, 2), 0, 1, z(4, 2, 8), z(4, 2, 8), z(4, 2, 32), z(4, 2, 8), z(2, 8))
        torch_native_op.native_lstm2_grad_multi([a, b])


@pytest.mark.parametrize("T,B,n,dtype", [(40, 16, 256, "bf16"), (12, 9, 1024, "f32"), (10, 40, 128, "f32")])
def test_bwd_bounded_wait_expires_cleanly(T, B, n, dtype):
    """A wait bound of zero ticks forced from the host: the persistent gradient kernel (the ordinary variant, the one
    with half of W in LDS, and a batch in several groups) must still drain; the status call then reports success
    (nobody had to wait) or the abort, and the next ordinary call on the same workspace is unaffected."""
    from _gpu_util import env

    announce("bwd bounded wait", T, B, n, dtype)
    X, W, y0, c0, i = random_problem(77 + n, T, B, n)
    rng = numpy.random.default_rng(78)
    DY = rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32)
    Dd = rng.normal(0, 1.0, (B, n)).astype(numpy.float32)
    op = get_op()
    Xd, Wd, y0d, DYd = (to_dev(a, dtype) for a in (X, W, y0, DY))
    c0d, id_, Ddd = (to_dev(a, "f32") for a in (c0, i, Dd))
    Y, C, H, d = op(Xd, Wd, y0d, c0d, id_, 0, 1)
    cabi = lib.load()
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    DX = torch.empty((T, B, 4 * n), dtype=act, device="cuda:0")
    DW = torch.empty((n, 4 * n), dtype=torch.float32, device="cuda:0")
    Dy0 = torch.empty((B, n), dtype=act, device="cuda:0")
    Dc0 = torch.empty((B, n), dtype=torch.float32, device="cuda:0")
    ws = torch.empty((max(int(cabi.rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dt)), 256),), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream

    def call():
        return cabi.rtn_native_lstm2_bwd(
            Wd.data_ptr(), y0d.data_ptr(), c0d.data_ptr(), id_.data_ptr(), 0, 1, Y.data_ptr(), C.data_ptr(), H.data_ptr(),
            DYd.data_ptr(), Ddd.data_ptr(), DX.data_ptr(), DW.data_ptr(), Dy0.data_ptr(), Dc0.data_ptr(), T, B, n, dt,
            ws.data_ptr(), ws.numel(), stream,
        )  # fmt: skip

    with env(RTN_LSTM2_TIMEOUT_TICKS=0, RTN_LSTM2_BWD_KERNEL=2):
        assert call() == 0
    status = cabi.rtn_native_lstm2_fwd_status(ws.data_ptr(), stream)
    assert status in (lib.RTN_OK, lib.RTN_ERR_ABORTED)
    if status == lib.RTN_ERR_ABORTED:
        # visible without the status query too: NaN where every caller looks
        assert bool(torch.isnan(Dc0).any()) and bool(torch.isnan(Dy0.float()).any()), "no NaN marks after an expired wait"
    assert call() == 0
    assert cabi.rtn_native_lstm2_fwd_status(ws.data_ptr(), stream) == lib.RTN_OK
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    want = oracle.native_lstm2_bwd(f(Xd), f(Wd), f(y0d), c0, i, 0, 1, f(Y), f(C), f(H), f(DYd), Dd, dtype=numpy.float64)
    for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), (DX, DW, Dy0, Dc0), want):
        assert _rel_to_max(f(a), b) <= (2e-5 if dtype == "f32" else 2e-2), name


@pytest.mark.parametrize("T,B,n,dtype", [(10, 8, 128, "bf16"), (8, 5, 100, "f32"), (6, 3, 20, "f32")])
def test_forward_and_gradient_recorded_into_a_callers_graph(T, B, n, dtype):
    """A training step under stream capture: forward op and gradient op (one launch per frame plus the rocBLAS weight
    gradient) are recorded into the caller's graph after one eager run (which creates the library's rocBLAS handle).
    The graph is replayed three times with new inputs and eager work in between; every replay must agree with the
    eager gradient op (another decomposition: equal up to rounding) and with the oracle."""
    announce("captured training step", T, B, n, dtype)
    op = get_op()
    rng = numpy.random.default_rng(5)
    problems = [random_problem(1200 + k, T, B, n) for k in range(3)]
    grads_in = [(rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32), rng.normal(0, 1.0, (B, n)).astype(numpy.float32)) for _ in range(3)]
    X, W, y0, c0, i = problems[0]
    Xd, Wd, y0d, DYd = (to_dev(a, dtype) for a in (X, W, y0, grads_in[0][0]))
    c0d, id_, Ddd = (to_dev(a, "f32") for a in (c0, i, grads_in[0][1]))

    def step():
        Y, C, H, d = op(Xd, Wd, y0d, c0d, id_, 0, 1)
        return (Y, C, H, d), torch_native_op.native_lstm2_grad(Wd, y0d, c0d, id_, 0, 1, Y, C, H, DYd, Ddd)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # eager warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        fwd_out, grad_out = step()
    f = lambda t: t.float().cpu().numpy().astype(numpy.float64)  # noqa: E731
    tol = 2e-5 if dtype == "f32" else 2e-2
    for k in range(3):
        Xk, Wk, y0k, c0k, ik = problems[k]
        for dst, src, dt in ((Xd, Xk, dtype), (Wd, Wk, dtype), (y0d, y0k, dtype), (DYd, grads_in[k][0], dtype), (c0d, c0k, "f32"),
                             (id_, ik, "f32"), (Ddd, grads_in[k][1], "f32")):  # fmt: skip
            dst.copy_(to_dev(src, dt))
        graph.replay()
        torch.cuda.synchronize()
        got_f = [t.clone() for t in fwd_out]
        got_g = [t.clone() for t in grad_out]
        eager_f, eager_g = step()
        torch.cuda.synchronize()
        for name, a, b in zip("YCHd", got_f, eager_f):
            assert torch.equal(a, b), (k, name)
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got_g, eager_g):
            assert _rel_to_max(f(a), f(b)) <= tol, (k, name, "against the eager op")
        want = oracle.native_lstm2_bwd(f(Xd), f(Wd), f(y0d), c0k, ik, 0, 1, f(got_f[0]), f(got_f[1]), f(got_f[2]), f(DYd), grads_in[k][1], dtype=numpy.float64)
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), got_g, want):
            assert _rel_to_max(f(a), b) <= tol, (k, name, "against the oracle")


def test_gradient_from_two_host_threads_on_their_own_streams():
    """Two host threads, each with a stream of its own, run forward and gradient at the same time (the weight-gradient
    GEMMs go through a rocBLAS handle per thread, so neither can have its stream changed by the other).  Every result must
    equal what the main thread computes alone."""
    import threading

    announce("bwd from two threads")
    op = get_op()
    shapes = [(14, 6, 128, "bf16"), (11, 5, 160, "f32")]
    inputs, want = [], []
    for k, (T, B, n, dtype) in enumerate(shapes):
        X, W, y0, c0, i = random_problem(640 + k, T, B, n)
        rng = numpy.random.default_rng(650 + k)
        DY = rng.normal(0, 1.0, (T, B, n)).astype(numpy.float32)
        Dd = rng.normal(0, 1.0, (B, n)).astype(numpy.float32)
        Xd, Wd, y0d, DYd = (to_dev(a, dtype) for a in (X, W, y0, DY))
        c0d, id_, Ddd = (to_dev(a, "f32") for a in (c0, i, Dd))
        inputs.append((Xd, Wd, y0d, c0d, id_, DYd, Ddd))
        Y, C, H, _ = op(Xd, Wd, y0d, c0d, id_, 0, 1)
        want.append(torch_native_op.native_lstm2_grad(Wd, y0d, c0d, id_, 0, 1, Y, C, H, DYd, Ddd))
    torch.cuda.synchronize()
    results, errors = {}, []

    def work(k):
        try:
            Xd, Wd, y0d, c0d, id_, DYd, Ddd = inputs[k]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for r in range(6):
                    Y, C, H, _ = op(Xd, Wd, y0d, c0d, id_, 0, 1)
                    results[(k, r)] = torch_native_op.native_lstm2_grad(Wd, y0d, c0d, id_, 0, 1, Y, C, H, DYd, Ddd)
            stream.synchronize()
        except Exception as exc:  # noqa: BLE001
            errors.append((k, exc))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for (k, r), grads in sorted(results.items()):
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), grads, want[k]):
            if name == "DW":  # rocBLAS may sum in another order from run to run
                assert _rel_to_max(a.double().cpu().numpy(), b.double().cpu().numpy()) <= 1e-5, (k, r, name)
            else:
                assert torch.equal(a, b), "thread %i, round %i: %s differs from the single-threaded result" % (k, r, name)
