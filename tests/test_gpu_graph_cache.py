"""
The library-owned graphs behind GRAPH mode and behind the per-frame launches of the gradient entries.

A graph is kept per shape, element type, plan and device, never per address: a call with other buffers of a known shape
writes its parameter block into the kept graph's kernel nodes instead of building a new graph.  More shapes than the cache
holds push the least recently used graph out; it is destroyed only once its last launch has completed.  Whatever the
cache does, the results must be, bit for bit, those of plain per-step launches.
"""

from __future__ import annotations

import numpy
import pytest
import torch

from returnn_amd import lib, torch_native_op
from _gpu_util import announce, env, get_op, random_problem, to_dev

pytestmark = pytest.mark.gpu

# More shapes than the cache keeps (8), none of them used by another test: generic kernels (n <= 32), the matrix-core kernel
# per step with and without batch tiles, both element types.
SHAPES = [
    (7, 3, 96, "f32"), (9, 5, 160, "bf16"), (6, 2, 224, "f32"), (11, 4, 24, "f32"), (8, 19, 96, "bf16"),
    (5, 33, 160, "f32"), (10, 1, 288, "bf16"), (7, 6, 12, "bf16"), (6, 7, 352, "f32"), (9, 2, 416, "bf16"),
]  # fmt: skip


def _forward(problem, dtype, mode, keep):
    """One forward call through the C ABI on freshly allocated buffers, which `keep` holds on to (so that the next call
    cannot get the same addresses)."""
    cabi = lib.load()
    X, W, y0, c0, i = problem
    T, B = i.shape
    n = y0.shape[1]
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    md = lib.MODES[mode]
    ins = [to_dev(X, dtype), to_dev(W, dtype), to_dev(y0, dtype), to_dev(c0, "f32"), to_dev(i, "f32")]
    outs = [torch.full((T, B, n), float("nan"), dtype=act, device="cuda:0"), torch.full((T, B, n), float("nan"), device="cuda:0"),
            torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0"), torch.full((B, n), float("nan"), device="cuda:0")]  # fmt: skip
    ws = torch.empty((max(lib.workspace_bytes(T, B, n, dt, md), 256),), dtype=torch.uint8, device="cuda:0")
    keep.extend(ins + outs + [ws])
    lib.check(cabi.rtn_native_lstm2_fwd(
        *(t.data_ptr() for t in ins), 0, 1, *(t.data_ptr() for t in outs), T, B, n, dt, md, ws.data_ptr(), ws.numel(),
        torch.cuda.current_stream().cuda_stream,
    ))  # fmt: skip
    return outs


def _same(got, want, what):
    for name, a, b in zip("YCHd", got, want):
        a, b = a.float().cpu().numpy(), b.float().cpu().numpy()
        assert numpy.isfinite(a).all(), (what, name)
        assert numpy.array_equal(a, b), "%s: %s differs from per-step launches" % (what, name)


def test_more_shapes_than_the_cache_holds_and_other_buffers():
    announce("graph cache: shapes and buffers")
    get_op()
    keep = []
    before = lib.graph_cache_stats()
    problems = {}
    for k, (T, B, n, dtype) in enumerate(SHAPES):
        problems[k] = [random_problem(4000 + 10 * k + r, T, B, n) for r in range(3)]
    # first visit of every shape: ten graphs built, at most eight kept
    for k, (T, B, n, dtype) in enumerate(SHAPES):
        assert "mode=graph" in lib.describe_plan(T, B, n, lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32, lib.MODE_GRAPH)
        got = _forward(problems[k][0], dtype, "graph", keep)
        want = _forward(problems[k][0], dtype, "stepwise", keep)
        torch.cuda.synchronize()
        _same(got, want, "first visit of %r" % (SHAPES[k],))
    after = lib.graph_cache_stats()
    assert after["built"] - before["built"] == len(SHAPES), (before, after)
    assert after["kept"] <= 8
    # the last eight shapes again, on other buffers with other data: no new graph, the kept one is re-aimed
    for k in range(2, len(SHAPES)):
        T, B, n, dtype = SHAPES[k]
        for r in (1, 2):
            got = _forward(problems[k][r], dtype, "graph", keep)
            want = _forward(problems[k][r], dtype, "stepwise", keep)
            torch.cuda.synchronize()
            _same(got, want, "visit %i of %r" % (r + 1, SHAPES[k]))
    again = lib.graph_cache_stats()
    assert again["built"] == after["built"], "a known shape on other buffers built a new graph: %r -> %r" % (after, again)
    assert again["retargeted"] - after["retargeted"] >= 2 * (len(SHAPES) - 2), (after, again)
    # the two shapes pushed out come back: built again, and what they push out is destroyed once it has run
    for k in (0, 1):
        T, B, n, dtype = SHAPES[k]
        got = _forward(problems[k][1], dtype, "graph", keep)
        want = _forward(problems[k][1], dtype, "stepwise", keep)
        torch.cuda.synchronize()
        _same(got, want, "return of %r" % (SHAPES[k],))
    end = lib.graph_cache_stats()  # (the query itself destroys what has completed)
    assert end["built"] == again["built"] + 2
    assert end["kept"] <= 8 and end["retiring"] == 0
    assert end["destroyed"] - before["destroyed"] >= 4, (before, end)


def test_same_graph_back_to_back_on_other_buffers_without_waiting():
    """Launches of one kept graph queued behind each other, every one on other buffers, with no synchronisation in
    between: a launch must keep the arguments it was queued with."""
    announce("graph cache: back to back")
    get_op()
    T, B, n, dtype = 12, 6, 192, "bf16"
    keep = []
    problems = [random_problem(4200 + r, T, B, n) for r in range(6)]
    got = [_forward(p, dtype, "graph", keep) for p in problems]
    want = [_forward(p, dtype, "stepwise", keep) for p in problems]
    torch.cuda.synchronize()
    for r in range(len(problems)):
        _same(got[r], want[r], "queued launch %i" % r)


def test_two_streams_share_shapes_without_waiting_for_each_other():
    """Two streams run the same shapes at the same time, each on its own buffers, over more shapes than the cache holds,
    with no synchronisation until the end.  A kept graph belongs to the stream it was first launched on, so one stream's
    call never rewrites or retires an executable graph that the other stream may still be running."""
    announce("graph cache: two streams")
    get_op()
    keep, got, want = [], {}, {}
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    problems = {(k, q): random_problem(4500 + 10 * k + q, *SHAPES[k][:3]) for k in range(len(SHAPES)) for q in range(2)}
    torch.cuda.synchronize()
    before = lib.graph_cache_stats()
    for rnd in range(2):  # the second round meets graphs pushed out by the first
        for k, (T, B, n, dtype) in enumerate(SHAPES):
            for q, st in enumerate(streams):
                with torch.cuda.stream(st):
                    got[(rnd, k, q)] = _forward(problems[(k, q)], dtype, "graph", keep)
    torch.cuda.synchronize()
    for k, (T, B, n, dtype) in enumerate(SHAPES):
        for q in range(2):
            want[(k, q)] = _forward(problems[(k, q)], dtype, "stepwise", keep)
    torch.cuda.synchronize()
    for (rnd, k, q), outs in got.items():
        _same(outs, want[(k, q)], "round %i shape %r stream %i" % (rnd, SHAPES[k], q))
    after = lib.graph_cache_stats()
    assert after["built"] - before["built"] >= 2 * len(SHAPES), (before, after)  # one graph per shape and stream
    assert after["kept"] <= 8 and after["retiring"] == 0, after


@pytest.mark.parametrize("T,B,n,dtype", [(9, 5, 128, "bf16"), (7, 3, 20, "f32")])
def test_gradient_graph_on_other_buffers(T, B, n, dtype):
    """The per-frame launches of the gradient entry go through the same cache: other buffers of a known shape reuse the
    kept graph, and the results equal those of the same launches made directly."""
    announce("graph cache: gradient", T, B, n, dtype)
    op = get_op()
    rng = numpy.random.default_rng(9)
    keep, results = [], {}
    for variant in ("graph", "direct"):
        for r in range(3):
            X, W, y0, c0, i = random_problem(4300 + r, T, B, n)
            DY = numpy.random.default_rng(50 + r).normal(0, 1.0, (T, B, n)).astype(numpy.float32)
            Dd = numpy.random.default_rng(60 + r).normal(0, 1.0, (B, n)).astype(numpy.float32)
            Xd, Wd, y0d, DYd = (to_dev(a, dtype) for a in (X, W, y0, DY))
            c0d, id_, Ddd = (to_dev(a, "f32") for a in (c0, i, Dd))
            Y, C, H, _ = op(Xd, Wd, y0d, c0d, id_, 0, 1)
            with env(RTN_LSTM2_BWD_KERNEL=1, RTN_LSTM2_BWD_NO_GRAPH=1 if variant == "direct" else None):
                before = lib.graph_cache_stats()
                grads = torch_native_op.native_lstm2_grad(Wd, y0d, c0d, id_, 0, 1, Y, C, H, DYd, Ddd)
                after = lib.graph_cache_stats()
            keep.extend([Xd, Wd, y0d, DYd, c0d, id_, Ddd, Y, C, H, *grads])
            if variant == "graph" and r > 0:
                assert after["built"] == before["built"], "other buffers of a known shape built a new gradient graph"
            results[(variant, r)] = grads
    del rng
    torch.cuda.synchronize()
    for r in range(3):
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), results[("graph", r)], results[("direct", r)]):
            assert torch.equal(a, b), "%s of problem %i: graph launches differ from direct launches" % (name, r)
