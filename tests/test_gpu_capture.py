"""
The persistent kernels under stream capture (the reference's whole-step graph capture, returnn/torch/util/graph_capture.py:
1-80, records its ops as launches on the capture stream).  A cooperative launch cannot be recorded through the stream API;
the library adds the kernel node to the capturing graph itself, with the cooperative attribute, or as an ordinary kernel
node where that is refused or not wanted.  Either way a replay must return, bit for bit, what the eager call returns, for
new inputs too, and must cost about what the eager call costs.
"""

from __future__ import annotations

import numpy
import pytest
import torch

from returnn_amd import lib, torch_native_op
from _gpu_util import announce, env, get_op, random_problem, to_dev

pytestmark = pytest.mark.gpu


def _timed(fn, reps=5):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


@pytest.mark.parametrize("node", ["cooperative", "plain"])
def test_forward_at_benchmark_shape(node):
    announce("persistent forward under capture", node)
    T, B, n, dtype = 1000, 32, 1024, "bf16"
    op = get_op()
    problems = [random_problem(1500 + k, T, B, n) for k in range(2)]
    X, W, y0, c0, i = problems[0]
    args = [to_dev(X, dtype), to_dev(W, dtype), to_dev(y0, dtype), to_dev(c0, "f32"), to_dev(i, "f32")]
    want = op(*args, 0, 1)
    t_eager = _timed(lambda: op(*args, 0, 1))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with env(RTN_LSTM2_CAPTURE_NODE=node):
        with torch.cuda.graph(graph, stream=side):
            got = op(*args, 0, 1)
    report = lib.capture_report()
    print("[capture]", report, flush=True)
    if node == "cooperative":
        assert "refused" not in report, report  # (the runtime of this image takes the attribute; a refusal would fall back)
    graph.replay()
    torch.cuda.synchronize()
    for name, a, b in zip("YCHd", got, want):
        assert torch.equal(a, b), "%s: replay differs from the eager call (%s node)" % (name, node)
    t_replay = _timed(graph.replay)
    print("[capture] eager %.3f ms, replay %.3f ms" % (t_eager, t_replay), flush=True)
    assert t_replay <= 1.3 * t_eager, (t_replay, t_eager)
    # new inputs in the captured buffers, eager work of the program in between
    X2, W2, y02, c02, i2 = problems[1]
    for dst, src, dt in zip(args, (X2, W2, y02, c02, i2), (dtype, dtype, dtype, "f32", "f32")):
        dst.copy_(to_dev(src, dt))
    want2 = op(*args, 0, 1)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip("YCHd", got, want2):
            assert torch.equal(a, b), "%s: replay with new inputs differs (%s node)" % (name, node)
        _ = (args[0].float() * 2).sum().item()  # eager work between replays


def test_per_step_recording_still_available():
    announce("RTN_LSTM2_CAPTURE=steps")
    T, B, n, dtype = 40, 8, 256, "f32"
    op = get_op()
    X, W, y0, c0, i = random_problem(1600, T, B, n)
    args = [to_dev(a, "f32") for a in (X, W, y0, c0, i)]
    want = op(*args, 0, -1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    before = lib.capture_report()
    with env(RTN_LSTM2_CAPTURE="steps"):
        with torch.cuda.graph(graph, stream=side):
            got = op(*args, 0, -1)
    assert lib.capture_report() == before, "a persistent kernel was recorded although per-step launches were asked for"
    for _ in range(2):
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip("YCHd", got, want):
            assert torch.equal(a, b), name


def test_training_step_at_benchmark_shape():
    """Forward and gradient of both directions (the multi-call entries: one persistent kernel each) recorded into one
    graph after an eager run; replays equal the eager results and cost about the same."""
    announce("persistent forward + gradient under capture")
    T, B, n, dtype = 400, 32, 1024, "bf16"
    get_op()
    rng = numpy.random.default_rng(3)
    X, W, y0, c0, i = random_problem(1700, T, B, n)
    Xd, y0d = to_dev(X, dtype), to_dev(y0, dtype)
    Wd = [to_dev(W, dtype), to_dev(numpy.ascontiguousarray(W[::-1]), dtype)]
    c0d, id_ = to_dev(c0, "f32"), to_dev(i, "f32")
    DY = [to_dev(rng.normal(0, 1, (T, B, n)).astype(numpy.float32), dtype) for _ in range(2)]
    Dd = [to_dev(rng.normal(0, 1, (B, n)).astype(numpy.float32), "f32") for _ in range(2)]

    def step():
        fw = torch_native_op.native_lstm2_multi([(Xd, Wd[0], y0d, c0d, id_, 0, 1), (Xd, Wd[1], y0d, c0d, id_, 0, -1)])
        calls = [(Wd[k], y0d, c0d, id_, 0, (1, -1)[k], fw[k][0], fw[k][1], fw[k][2], DY[k], Dd[k]) for k in range(2)]
        return fw, torch_native_op.native_lstm2_grad_multi(calls)

    fw_want, bw_want = step()  # eager (also creates the rocBLAS handle of this thread)
    t_eager = _timed(step, reps=3)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        fw_got, bw_got = step()
    print("[capture]", lib.capture_report(), flush=True)
    graph.replay()
    torch.cuda.synchronize()
    for k in range(2):
        for name, a, b in zip("YCHd", fw_got[k], fw_want[k]):
            assert torch.equal(a, b), (k, name)
        for name, a, b in zip(("DX", "DW", "Dy0", "Dc0"), bw_got[k], bw_want[k]):
            if name == "DW":  # rocBLAS may sum in another order
                scale = float(b.abs().max())
                assert float((a - b).abs().max()) <= 1e-5 * scale, (k, name)
            else:
                assert torch.equal(a, b), (k, name)
    t_replay = _timed(graph.replay, reps=3)
    print("[capture] training step: eager %.3f ms, replay %.3f ms" % (t_eager, t_replay), flush=True)
    assert t_replay <= 1.3 * t_eager, (t_replay, t_eager)
