"""
XCD-local plans of the persistent kernel: every batch group on one XCD, the hidden state handed over through that
XCD's L2.  Whatever the plan, an op call must return bit for bit what per-step launches return (which the parity
tests pin against the oracle), the kernel must find its groups where the plan put them, and when they are not there
(forced here with a wrong XCD count) it must notice and still return the same bits.
"""

from __future__ import annotations

import numpy
import pytest
import torch

from returnn_amd import lib
from _gpu_util import announce, env, get_op, random_problem, to_dev

pytestmark = pytest.mark.gpu


def _run(problems, dtype, mode, starts_steps):
    """All problems (one shape) through the multi-call entry; returns outputs, the plan text and the status words."""
    get_op()
    cabi = lib.load()
    T, B = problems[0][4].shape
    n = problems[0][2].shape[1]
    count = len(problems)
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    md = lib.MODES[mode]
    keep, outs = [], []
    calls = (lib.Lstm2Call * count)()
    for k, (X, W, y0, c0, i) in enumerate(problems):
        d_in = [to_dev(X, dtype), to_dev(W, dtype), to_dev(y0, dtype), to_dev(c0, "f32"), to_dev(i, "f32")]
        o = [torch.full((T, B, n), float("nan"), dtype=act, device="cuda:0"), torch.full((T, B, n), float("nan"), device="cuda:0"),
             torch.full((T, B, 4 * n), float("nan"), dtype=act, device="cuda:0"), torch.full((B, n), float("nan"), device="cuda:0")]
        keep.append(d_in)
        outs.append(o)
        start, step = starts_steps[k % len(starts_steps)]
        calls[k] = lib.Lstm2Call(*(t.data_ptr() for t in d_in), start, step, *(t.data_ptr() for t in o))
    ws = torch.zeros((max(cabi.rtn_native_lstm2_fwd_multi_workspace_bytes(count, T, B, n, dt, md), 256),), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    lib.check(cabi.rtn_native_lstm2_fwd_multi(calls, count, T, B, n, dt, md, ws.data_ptr(), ws.numel(), stream))
    lib.check(cabi.rtn_native_lstm2_fwd_multi_status(ws.data_ptr(), count, T, B, n, dt, md, stream))
    torch.cuda.synchronize()
    plan = lib.describe_multi_plan(count, T, B, n, dt, md)
    each = ws.numel() // count
    words = [ws[k * each : k * each + 8].view(torch.int32).cpu().tolist() for k in range(count)]
    return [[t.float().cpu().numpy() for t in o] for o in outs], plan, words


CASES = [
    # T, B, n, dtype, count: what the XCD-local plan looks like on 8 XCDs of 32 CUs
    (40, 32, 1024, "bf16", 2),   # the benchmark pair: 2 x 4 groups of 8 rows, half-tile pointwise part
    (30, 32, 1024, "bf16", 1),   # 8 groups of 4 rows
    (24, 128, 1024, "bf16", 1),  # 16 rows per group: whole tiles
    (25, 64, 512, "f32", 1),     # float32, 16 cells per workgroup
    (20, 200, 256, "bf16", 1),   # 13 rows per group (16 groups of 16 workgroups) or 25 (two batch tiles)
    (18, 32, 768, "bf16", 1),    # 24 workgroups per group: part of an XCD
    (22, 5, 64, "f32", 1),       # two groups per XCD
    (15, 6, 96, "bf16", 1),      # 3 macro steps of the contraction over 4 wavefronts: one wavefront without a share
    (13, 8, 160, "bf16", 2),     # 5 macro steps: the paired loads of h end on an odd step
    (12, 7, 352, "bf16", 1),     # 11 macro steps
    (11, 3, 224, "f32", 1),      # 14 macro steps in float32
    (16, 3, 32, "f32", 1),       # four groups per XCD
    (21, 9, 512, "bf16", 3),     # three problems
]


@pytest.mark.parametrize("T,B,n,dtype,count", CASES)
def test_local_plan_equals_stepwise_and_spread(T, B, n, dtype, count):
    announce("xcd-local", T, B, n, dtype, count)
    problems = [random_problem(300 + k, T, B, n) for k in range(count)]
    ss = [(0, 1), (0, -1), (1, 2)]
    want, _, _ = _run(problems, dtype, "stepwise", ss)
    with env(RTN_LSTM2_LOCAL=1):
        got, plan, words = _run(problems, dtype, "auto", ss)
    assert "kernel=mfma_regw_xcd" in plan, plan
    for k in range(count):
        assert words[k][0] == 0 and words[k][1] == 0, "problem %i: status %r (word 1: XCDs a spread group was found on)" % (k, words[k][:2])
        for name, a, b in zip("YCHd", got[k], want[k]):
            assert numpy.isfinite(a).all(), name
            assert numpy.array_equal(a, b), "%s of problem %i differs from per-step launches (%s)" % (name, k, plan)
    with env(RTN_LSTM2_LOCAL=0):
        spread, plan_s, _ = _run(problems, dtype, "auto", ss)
    assert "kernel=mfma_regw_xcd" not in plan_s, plan_s
    for k in range(count):
        for name, a, b in zip("YCHd", spread[k], want[k]):
            assert numpy.array_equal(a, b), "%s of problem %i differs (%s)" % (name, k, plan_s)


def test_groups_found_on_several_xcds_fall_back_to_device_scope():
    """With half the true XCD count every group of the plan lands on two XCDs.  The kernel's check finds that out
    (status word 1 records the XCDs seen) and exchanges at device scope: same bits, no abort."""
    announce("xcd-local with a wrong XCD count")
    T, B, n = 30, 32, 1024
    problems = [random_problem(41, T, B, n)]
    want, _, _ = _run(problems, "bf16", "stepwise", [(0, 1)])
    with env(RTN_LSTM2_LOCAL=1, RTN_LSTM2_XCDS=4):
        got, plan, words = _run(problems, "bf16", "auto", [(0, 1)])
    assert "kernel=mfma_regw_xcd" in plan, plan
    assert words[0][0] == 0, "aborted"
    mask = words[0][1] & 0xFFFF
    assert bin(mask).count("1") >= 2, "expected a group spread over XCDs, saw mask %#x (%s)" % (mask, plan)
    for name, a, b in zip("YCHd", got[0], want[0]):
        assert numpy.array_equal(a, b), name


def test_local_plan_start_step_and_masks_with_holes():
    announce("xcd-local start/step/holes")
    T, B, n = 26, 12, 256
    X, W, y0, c0, i = random_problem(77, T, B, n)
    rng = numpy.random.default_rng(5)
    i = (rng.uniform(size=(T, B)) < 0.7).astype(numpy.float32)  # holes anywhere, not only right padding
    for start, step in [(0, 1), (3, 1), (0, -1), (2, -3), (1, 4)]:
        want, _, _ = _run([(X, W, y0, c0, i)], "f32", "stepwise", [(start, step)])
        with env(RTN_LSTM2_LOCAL=1):
            got, plan, words = _run([(X, W, y0, c0, i)], "f32", "auto", [(start, step)])
        assert "kernel=mfma_regw_xcd" in plan and words[0][:2] == [0, 0], (plan, words)
        for name, a, b in zip("YCHd", got[0], want[0]):
            assert numpy.array_equal(a, b), "%s start=%i step=%i" % (name, start, step)


@pytest.mark.parametrize("delay,inc", [(0, 0), (64, 0), (0, 2), (20, 2)])
def test_first_read_delay_only_moves_time(delay, inc):
    """The delay between a step's exchange stores and the first read of the next step (fixed inside an XCD, adaptive
    across XCDs) decides how often a read has to be repeated, never what is read: any setting gives the same bits."""
    announce("first-read delay", delay, inc)
    T, B, n, dtype = 30, 16, 512, "bf16"
    problems = [random_problem(900 + k, T, B, n) for k in range(2)]
    ss = [(0, 1), (0, -1)]
    want, _, _ = _run(problems, dtype, "stepwise", ss)
    for local in (1, 0):
        with env(RTN_LSTM2_LOCAL=local, RTN_LSTM2_POLL_DELAY=delay, RTN_LSTM2_DELAY_INC=inc):
            got, plan, words = _run(problems, dtype, "auto", ss)
        assert ("kernel=mfma_regw_xcd" in plan) == bool(local), plan
        for k in range(len(problems)):
            assert words[k][0] == 0, (plan, words[k])
            for name, a, b in zip("YCHd", got[k], want[k]):
                assert numpy.array_equal(a, b), (plan, k, name)
