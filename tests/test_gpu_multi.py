"""
The multi-call entry (several op calls of one shape per entry, fused into one launch when they fit) must return,
for every element, bit for bit what a single call of the op returns for the same arguments -- the single call is
what the parity tests pin against the oracle.
"""

from __future__ import annotations

import pytest
import torch

from returnn_amd import lib, synthetic, torch_native_op
from _gpu_util import announce, env, get_op, random_problem, to_dev

pytestmark = pytest.mark.gpu


def _single(args, dtype, mode="auto"):
    op = get_op(mode)
    return op(*args)


def _args(seed, T, B, n, dtype, start, step, **kw):
    X, W, y0, c0, i = random_problem(seed, T, B, n, **kw)
    return (to_dev(X, dtype), to_dev(W, dtype), to_dev(y0, dtype), to_dev(c0, "f32"), to_dev(i, "f32"), start, step)


def _assert_same(multi_out, single_out, what):
    for name, a, b in zip("YCHd", multi_out, single_out):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.equal(a, b), "%s: %s differs, max |diff| = %g" % (what, name, float((a.float() - b.float()).abs().max()))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize(
    "T,B,n,count",
    [(12, 16, 64, 2), (7, 32, 256, 2), (9, 5, 128, 3), (6, 40, 512, 4), (5, 8, 96, 6), (6, 3, 20, 2), (5, 32, 1024, 2), (6, 9, 100, 2), (4, 7, 72, 3),
     (4, 300, 512, 2)],  # (each call in several persistent launches in turn, the last one on fewer groups)
)
def test_multi_equals_single(T, B, n, count, dtype):
    announce("multi vs single", T, B, n, count, dtype)
    get_op()
    steps = [(0, 1), (0, -1), (1, 2), (2, -1), (0, 1), (1, -2)]
    calls = [_args(100 + k, T, B, n, dtype, *steps[k % len(steps)]) for k in range(count)]
    outs = torch_native_op.native_lstm2_multi(calls)
    torch.cuda.synchronize()
    assert len(outs) == count
    for k in range(count):
        _assert_same(outs[k], _single(calls[k], dtype), "call %i" % k)


@pytest.mark.parametrize("mode", ["persistent", "graph", "stepwise"])
def test_multi_modes(mode):
    announce("multi modes", mode)
    get_op()
    calls = [_args(7, 10, 16, 128, "bf16", 0, 1), _args(8, 10, 16, 128, "bf16", 0, -1)]
    outs = torch_native_op.native_lstm2_multi(calls, mode=mode)
    for k in range(2):
        _assert_same(outs[k], _single(calls[k], "bf16", "stepwise"), "mode %s call %i" % (mode, k))


def test_multi_fused_and_sequential_agree():
    """Fusing is a scheduling choice: switching it off gives the same bits."""
    announce("multi fused vs sequential")
    get_op()
    calls = [_args(21, 40, 32, 256, "bf16", 0, 1), _args(22, 40, 32, 256, "bf16", 0, -1)]
    fused = torch_native_op.native_lstm2_multi(calls)
    with env(RTN_LSTM2_NO_FUSE=1):
        seq = torch_native_op.native_lstm2_multi(calls)
    for k in range(2):
        _assert_same(fused[k], seq[k], "call %i" % k)


def test_multi_pair_cfg3_shape():
    """The bidirectional pair at the benchmark's width and batch (shortened), through the C ABI with poisoned outputs."""
    announce("multi pair cfg3 shape")
    get_op()
    cabi = lib.load()
    p = synthetic.make_config("cfg3", T=60)
    T, B, n = p.T, p.B, p.n
    X, W, y0 = (to_dev(a, "bf16") for a in (p.X, p.W, p.y0))
    c0, msk = to_dev(p.c0, "f32"), to_dev(p.i, "f32")
    arr = (lib.Lstm2Call * 2)()
    outs = []
    for k, step in enumerate((1, -1)):
        Y = torch.full((T, B, n), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        C = torch.full((T, B, n), float("nan"), device="cuda:0")
        H = torch.full((T, B, 4 * n), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        d = torch.full((B, n), float("nan"), device="cuda:0")
        outs.append((Y, C, H, d))
        arr[k] = lib.Lstm2Call(X.data_ptr(), W.data_ptr(), y0.data_ptr(), c0.data_ptr(), msk.data_ptr(), 0, step,
                               Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr())  # fmt: skip
    nbytes = cabi.rtn_native_lstm2_fwd_multi_workspace_bytes(2, T, B, n, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert nbytes >= 2 * lib.workspace_bytes(T, B, n, lib.DTYPE_BF16, lib.MODE_AUTO) and nbytes % 2 == 0
    ws = torch.empty((nbytes,), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    lib.check(cabi.rtn_native_lstm2_fwd_multi(arr, 2, T, B, n, lib.DTYPE_BF16, lib.MODE_AUTO, ws.data_ptr(), ws.numel(), stream))
    lib.check(cabi.rtn_native_lstm2_fwd_multi_status(ws.data_ptr(), 2, T, B, n, lib.DTYPE_BF16, lib.MODE_AUTO, stream))
    for k, step in enumerate((1, -1)):
        _assert_same(outs[k], _single((X, W, y0, c0, msk, 0, step), "bf16"), "step %i" % step)
    # too small a workspace is refused before anything is enqueued
    rc = cabi.rtn_native_lstm2_fwd_multi(arr, 2, T, B, n, lib.DTYPE_BF16, lib.MODE_AUTO, ws.data_ptr(), ws.numel() // 2, stream)
    assert rc == lib.RTN_ERR_WORKSPACE and "workspace" in lib.last_error()


def test_multi_edge_cases():
    announce("multi edge cases")
    get_op()
    cabi = lib.load()
    assert torch_native_op.native_lstm2_multi([]) == []
    assert cabi.rtn_native_lstm2_fwd_multi(None, 0, 5, 2, 32, 0, 0, None, 0, None) == lib.RTN_OK
    assert cabi.rtn_native_lstm2_fwd_multi(None, 2, 5, 2, 32, 0, 0, None, 0, None) == lib.RTN_ERR_ARG
    # T == 0: d = c0 for every call
    calls = [_args(3, 0, 4, 32, "f32", 0, 1, ragged=False), _args(4, 0, 4, 32, "f32", 0, 1, ragged=False)]
    outs = torch_native_op.native_lstm2_multi(calls)
    for c, o in zip(calls, outs):
        assert torch.equal(o[3], c[3]) and o[0].shape == (0, 4, 32)
    # mismatching shapes are refused
    with pytest.raises(RuntimeError, match="same T, B, n"):
        torch_native_op.native_lstm2_multi([_args(1, 4, 4, 32, "f32", 0, 1), _args(1, 5, 4, 32, "f32", 0, 1)])
    # a bad start in any element fails the whole entry
    with pytest.raises(RuntimeError, match="start"):
        torch_native_op.native_lstm2_multi([_args(1, 4, 4, 32, "f32", 0, 1), _args(1, 4, 4, 32, "f32", 9, 1)])
