"""
Nine more of the reference's native ops -- Chunking, UnChunking, SubtensorBatchedIndex, SparseToDense, MaxAndArgmaxSparse,
CrossEntropySoftmaxAndGradientZSparse, GetCtcFsaFastBwOp, GetCtcFsaFastBwPackedOp, FastBaumWelchPackedOp -- compiled for
gfx950 by this package's op loader from the reference's own op sources (tests/build_ref_ops.py) and run on the GPU.

The reference holds no numbers for these; its tests check them against library routines and numpy
(tests/test_TFNativeOp.py:1297-1560 chunking, :1629-1760 the CTC automaton against a CTC loss).  So do these:

* the array ops against what their documentation defines, written with numpy indexing (returnn/native_op.py:2321-2337,
  :2478-2486, :2655-2662, :2799-2804, :2880-2886, :2988-2995), plus the round trip chunk -> unchunk;
* the CTC automaton through the Baum-Welch op against ``torch.nn.functional.ctc_loss`` in float64 on the CPU: the loss
  value and, through its gradient, the soft alignment -- the reference's own check with torch's loss in place of
  TensorFlow's, on the reference's target sets (tests/test_TFNativeOp.py:1762-1885);
* the packed variants against the rectangular ops on the same sequences.

As in tests/test_gpu_ref_ops.py, what is under test is the loader (dialect header, generated entry point, in-place
inputs, host scalars, int32 arrays), on code that was not written for it.
"""

from __future__ import annotations

import json
import os

import numpy
import pytest
import torch

from returnn_amd import op_loader
import _fsa_numpy
from _gpu_util import announce

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OPS_DIR = os.path.join(ROOT, "tests", "_built_ref_ops")


def _built(*names):
    try:
        table = json.load(open(os.path.join(OPS_DIR, "ops.json")))
    except OSError:
        return False
    return all(n in table for n in names)


def needs(*names):
    return pytest.mark.skipif(
        not _built(*names), reason="tests/_built_ref_ops lacks %s (python tests/build_ref_ops.py, where the reference tree is)" % ", ".join(names)
    )


def _op(name):
    table = json.load(open(os.path.join(OPS_DIR, "ops.json")))
    return op_loader.CompiledOp.from_shared_object(name, table[name]["in_info"], table[name]["out_info"], os.path.join(OPS_DIR, name + ".so"))


def _dev(a):
    return torch.from_numpy(numpy.ascontiguousarray(a)).to("cuda:0")


def _host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def n_chunks_of(n_time, size, step):
    return max(n_time - size + step - 1, 0) // step + 1  # returnn/native_op.py:2326


def chunk_numpy(x, index, size, step):
    T, B, D = x.shape
    nc = n_chunks_of(T, size, step)
    out = numpy.zeros((size, B * nc, D), dtype=x.dtype)
    oindex = numpy.zeros((size, B * nc), dtype=x.dtype)
    for b in range(B):
        for c in range(nc):
            for k in range(size):
                t = step * c + k
                if t < T and index[t, b] > 0.1:
                    out[k, b * nc + c] = x[t, b]
                    oindex[k, b * nc + c] = 1
    return out, oindex


def unchunk_numpy(chunks, cindex, n_time, n_batch, size, step):
    D = chunks.shape[2]
    nc = chunks.shape[1] // n_batch
    total = numpy.zeros((n_time, n_batch, D), dtype=numpy.float64)
    count = numpy.zeros((n_time, n_batch))
    for b in range(n_batch):
        for c in range(nc):
            for k in range(size):
                t = step * c + k
                if t < n_time and cindex[k, b * nc + c] > 0.1:
                    total[t, b] += chunks[k, b * nc + c]
                    count[t, b] += 1
    out = total / numpy.maximum(count, 1)[:, :, None]
    return out, (count > 0).astype(numpy.float32), 1.0 / numpy.maximum(count, 1)


CHUNKINGS = [(2, 1), (2, 2), (4, 2), (4, 3), (4, 4), (10, 4), (20, 4)]  # tests/test_TFNativeOp.py:1385-1391


@needs("Chunking", "UnChunking")
@pytest.mark.parametrize("n_batch,n_dim,holes", [(1, 3, False), (3, 5, True)])
def test_chunking_and_unchunking(n_batch, n_dim, holes):
    announce("reference ops Chunking / UnChunking", n_batch, n_dim, holes)
    chunk, unchunk = _op("Chunking"), _op("UnChunking")
    rng = numpy.random.RandomState(3)
    T = 17
    x = rng.normal(size=(T, n_batch, n_dim)).astype(numpy.float32)
    index = numpy.ones((T, n_batch), dtype=numpy.float32)
    if holes:
        index[-2:, -1] = 0  # the last sequence is two frames shorter (tests/test_TFNativeOp.py:1399-1400)
    for size, step in CHUNKINGS:
        nc = n_chunks_of(T, size, step)
        params = numpy.array([size, step], dtype=numpy.float32)
        out_buf = torch.full((size, n_batch * nc, n_dim), 7.0, device="cuda:0")  # (the op overwrites every element)
        idx_buf = torch.full((size, n_batch * nc), 7.0, device="cuda:0")
        out, oindex = chunk(_dev(x), _dev(index), out_buf, idx_buf, _dev(params))
        assert out.data_ptr() == out_buf.data_ptr() and oindex.data_ptr() == idx_buf.data_ptr()  # worked in place
        want, want_index = chunk_numpy(x, index, size, step)
        assert numpy.array_equal(_host(out), want), (size, step)
        assert numpy.array_equal(_host(oindex), want_index), (size, step)
        # and back: the mean over the chunks that hold a frame is the frame
        back, bindex, factors = unchunk(
            out, oindex, torch.empty((T, n_batch, n_dim), device="cuda:0"), torch.empty((T, n_batch), device="cuda:0"),
            torch.empty((T, n_batch), device="cuda:0"), _dev(params))  # fmt: skip
        w_back, w_index, w_factors = unchunk_numpy(want, want_index, T, n_batch, size, step)
        numpy.testing.assert_allclose(_host(back), w_back, rtol=1e-6, atol=1e-7)
        assert numpy.array_equal(_host(bindex), w_index)
        numpy.testing.assert_allclose(_host(factors), w_factors, rtol=1e-6)
        numpy.testing.assert_allclose(_host(back), x * index[:, :, None], rtol=1e-6, atol=1e-6)
        assert numpy.array_equal(_host(bindex), index)


@needs("SubtensorBatchedIndex")
def test_subtensor_batched_index():
    announce("reference op SubtensorBatchedIndex")
    op = _op("SubtensorBatchedIndex")
    rng = numpy.random.RandomState(4)
    T, B, D = 11, 5, 7
    x = rng.normal(size=(T, B, D)).astype(numpy.float32)
    idx = rng.randint(-2, D + 2, size=(T, B))  # out-of-range indices are clipped (returnn/native_op.py:2695-2697)
    (y,) = op(_dev(x), _dev(idx.astype(numpy.float32)))
    want = numpy.take_along_axis(x, numpy.clip(idx, 0, D - 1)[:, :, None], axis=2)[:, :, 0]
    assert numpy.array_equal(_host(y), want)


def _sparse_case(rng, n_entries, n_batch, n_time, n_dim):
    """COO entries [n_entries, n_batch] with distinct (time, dim) cells per sequence and a mask with holes."""
    s0 = numpy.zeros((n_entries, n_batch), dtype=numpy.float32)
    s1 = numpy.zeros((n_entries, n_batch), dtype=numpy.float32)
    for b in range(n_batch):
        cells = rng.permutation(n_time * n_dim)[:n_entries]
        s0[:, b], s1[:, b] = cells // n_dim, cells % n_dim
    w = rng.uniform(0.1, 1.0, size=(n_entries, n_batch)).astype(numpy.float32)
    mask = (rng.uniform(size=(n_entries, n_batch)) > 0.25).astype(numpy.float32)
    return s0, s1, w, mask


@needs("SparseToDense")
def test_sparse_to_dense():
    announce("reference op SparseToDense")
    op = _op("SparseToDense")
    rng = numpy.random.RandomState(5)
    T, B, D, N = 6, 4, 9, 20
    s0, s1, w, mask = _sparse_case(rng, N, B, T, D)
    start = rng.normal(size=(T, B, D)).astype(numpy.float32)
    (W,) = op(_dev(start), _dev(s0), _dev(s1), _dev(w), _dev(mask))
    want = start.copy()
    for i in range(N):
        for b in range(B):
            if mask[i, b] > 0.1:
                want[int(s0[i, b]), b, int(s1[i, b])] += w[i, b]
    numpy.testing.assert_allclose(_host(W), want, rtol=1e-6)


@needs("MaxAndArgmaxSparse")
def test_max_and_argmax_sparse():
    announce("reference op MaxAndArgmaxSparse")
    op = _op("MaxAndArgmaxSparse")
    rng = numpy.random.RandomState(6)
    T, B, D, N = 5, 4, 8, 24
    s0, s1, w, mask = _sparse_case(rng, N, B, T, D)
    out_max, out_arg = op(_dev(s0), _dev(s1), _dev(w), _dev(mask), torch.full((T, B), -1.0, device="cuda:0"), torch.full((T, B), -1.0, device="cuda:0"))
    want_max, want_arg = numpy.full((T, B), -1.0, dtype=numpy.float32), numpy.full((T, B), -1.0, dtype=numpy.float32)
    for b in range(B):
        for i in range(N):  # (in this order: of equal weights the first one stays, returnn/native_op.py:2936-2939)
            t = int(s0[i, b])
            if mask[i, b] > 0.1 and w[i, b] > want_max[t, b]:
                want_max[t, b], want_arg[t, b] = w[i, b], s1[i, b]
    assert numpy.array_equal(_host(out_max), want_max)
    assert numpy.array_equal(_host(out_arg), want_arg)


@needs("CrossEntropySoftmaxAndGradientZSparse")
def test_cross_entropy_softmax_and_gradient_sparse():
    announce("reference op CrossEntropySoftmaxAndGradientZSparse")
    op = _op("CrossEntropySoftmaxAndGradientZSparse")
    rng = numpy.random.RandomState(7)
    T, B, D = 9, 3, 10
    N = T  # one target entry per frame, in any order: the op adds to a frame's cross entropy without atomics
    z = (3.0 * rng.normal(size=(T, B, D))).astype(numpy.float32)
    z_mask = numpy.ones((T, B), dtype=numpy.float32)
    z_mask[-1, 1] = 0
    s0 = numpy.stack([rng.permutation(T) for _ in range(B)], axis=1).astype(numpy.float32)
    s1 = rng.randint(0, D, size=(N, B)).astype(numpy.float32)
    w = rng.uniform(0.1, 1.0, size=(N, B)).astype(numpy.float32)
    s_mask = (rng.uniform(size=(N, B)) > 0.25).astype(numpy.float32)
    s_mask[(s0 == T - 1) & (numpy.arange(B)[None, :] == 1)] = 0  # no target where z is masked out
    ce, grad, max_z = op(_dev(z), _dev(z_mask), _dev(s0), _dev(s1), _dev(w), _dev(s_mask))
    z64 = z.astype(numpy.float64)
    sm = numpy.exp(z64 - z64.max(axis=2, keepdims=True))
    sm /= sm.sum(axis=2, keepdims=True)
    sm *= z_mask[:, :, None]
    target = numpy.zeros((T, B, D))
    for i in range(N):
        for b in range(B):
            if s_mask[i, b] > 0.1:
                target[int(s0[i, b]), b, int(s1[i, b])] += w[i, b]
    want_ce = -(target * numpy.log(numpy.maximum(sm, 1e-30))).sum(axis=2)
    numpy.testing.assert_allclose(_host(ce), want_ce, rtol=2e-5, atol=1e-6)
    numpy.testing.assert_allclose(_host(grad), sm - target, rtol=2e-5, atol=1e-6)
    inside = z_mask > 0.5
    assert numpy.array_equal(_host(max_z)[inside], z.max(axis=2)[inside])


CTC_TARGETS = [  # tests/test_TFNativeOp.py:1762-1885: targets, their lengths, classes including the blank
    ([[1, 3, 4, 2, 1, 0], [2, 6, 3, 4, 0, 0], [0, 3, 2, 0, 0, 0]], [6, 4, 3], 8),
    ([[1, 2, 4, 4, 1, 0], [2, 6, 3, 4, 0, 0], [3, 3, 0, 0, 0, 0], [5, 0, 0, 0, 0, 0]], [6, 4, 2, 1], 8),
    ([[0, 1]], [2], 3),
    ([[0]], [1], 2),
    ([[0, 1], [1, 0]], [2, 1], 3),
    ([[0, 1], [0, 0]], [2, 2], 3),
    ([[0], [1]], [1, 1], 3),
    ([[0, 0]], [2], 2),
]


def _ctc_inputs(targets, target_lens, n_classes):
    """Logits and frame counts as the reference's check makes them (tests/test_TFNativeOp.py:1640-1656)."""
    targets = numpy.array(targets, dtype=numpy.int32)
    target_lens = numpy.array(target_lens, dtype=numpy.int32)
    n_batch, n_target_time = targets.shape
    n_time = n_target_time * 3
    logits = numpy.random.RandomState(42).normal(size=(n_time, n_batch, n_classes)).astype(numpy.float32)
    lens = numpy.array([n_time, max(n_time - 4, (target_lens[1] if n_batch >= 2 else 0) + 1, 1), max(n_time - 5, 1), max(n_time - 5, 1)],
                       dtype=numpy.int32)[:n_batch]  # fmt: skip
    return targets, target_lens, logits, lens


def _torch_ctc(logits, lens, targets, target_lens, blank):
    """-log p(targets | logits) per sequence and the soft alignment, by torch's CTC loss in float64 on the CPU."""
    z = torch.tensor(logits, dtype=torch.float64, requires_grad=True)
    loss = torch.nn.functional.ctc_loss(
        torch.log_softmax(z, dim=2), torch.tensor(targets, dtype=torch.long), torch.tensor(lens, dtype=torch.long),
        torch.tensor(target_lens, dtype=torch.long), blank=blank, reduction="none")  # fmt: skip
    loss.sum().backward()
    soft_align = torch.softmax(z, dim=2) - z.grad  # d loss / d logits = softmax - alignment
    return loss.detach().numpy(), soft_align.detach().numpy()


def _check_against_ctc(fwdbwd, scores, logits, lens, targets, target_lens, blank):
    want_loss, want_align = _torch_ctc(logits, lens, targets, target_lens, blank)
    got_align = numpy.exp(-fwdbwd.astype(numpy.float64))
    for b in range(len(lens)):
        numpy.testing.assert_allclose(scores[: lens[b], b], want_loss[b], rtol=2e-5)  # the same in every frame
        numpy.testing.assert_allclose(got_align[: lens[b], b], want_align[: lens[b], b], rtol=2e-3, atol=2e-5)


@needs("GetCtcFsaFastBwOp", "FastBaumWelchOp")
@pytest.mark.parametrize("case", range(len(CTC_TARGETS)))
def test_ctc_automaton_through_baum_welch_equals_ctc_loss(case):
    targets, target_lens, logits, lens = _ctc_inputs(*CTC_TARGETS[case])
    announce("reference ops GetCtcFsaFastBwOp + FastBaumWelchOp", targets.shape, target_lens.tolist())
    make_fsa, baum_welch = _op("GetCtcFsaFastBwOp"), _op("FastBaumWelchOp")
    n_batch, n_target_time = targets.shape
    n_classes = logits.shape[2]
    blank = n_classes - 1
    n_edges = n_batch * (5 * (n_target_time - 1) + 10)  # returnn/tf/native_op.py:1416
    weights = torch.zeros((n_edges,), device="cuda:0")
    edges, start_end = make_fsa(_dev(targets), _dev(target_lens), blank, weights, 1)
    assert tuple(edges.shape) == (4, n_edges) and tuple(start_end.shape) == (2, n_batch)
    assert edges.dtype == torch.int32 and start_end.dtype == torch.int32
    n_states = int(_host(start_end)[1].max()) + 1  # returnn/tf/native_op.py:1312-1320
    index = (numpy.arange(logits.shape[0])[:, None] < lens[None, :]).astype(numpy.float32)
    am = -torch.log_softmax(torch.tensor(logits, dtype=torch.float64), dim=2).numpy().astype(numpy.float32)
    fwdbwd, scores = baum_welch(_dev(am), edges, weights, start_end, _dev(index), n_states)
    _check_against_ctc(_host(fwdbwd), _host(scores), logits, lens, targets, target_lens, blank)
    # the automaton itself, through the plain numpy recursion
    with numpy.errstate(invalid="ignore"):  # (frames behind a sequence's end: inf - inf)
        w_fb, w_score = _fsa_numpy.baum_welch(am.astype(numpy.float64), index, _host(edges), numpy.zeros(n_edges), _host(start_end), n_states)
    inside = index.astype(bool)
    numpy.testing.assert_allclose(_host(scores)[inside], w_score[inside], rtol=1e-5)


def _paths_by_enumeration(log_probs, target, blank, label_loop):
    """-log of the summed probability of all frame labellings of length T that give `target`: blanks removed, and with
    label_loop repeats of a label merged first (CTC); without it every non-blank frame is a label of its own (the
    recurrent neural aligner's topology).  By enumeration of all C^T labellings: for a handful of frames only."""
    import itertools

    T, C = log_probs.shape
    total = -numpy.inf
    for path in itertools.product(range(C), repeat=T):
        labels = [c for k, c in enumerate(path) if not (label_loop and k > 0 and path[k - 1] == c)]
        if [c for c in labels if c != blank] == list(target):
            total = numpy.logaddexp(total, sum(log_probs[t, c] for t, c in enumerate(path)))
    return -total


@needs("GetCtcFsaFastBwOp", "FastBaumWelchOp")
@pytest.mark.parametrize("label_loop", [True, False])
def test_ctc_automaton_with_and_without_label_loop_by_enumeration(label_loop):
    """Both topologies of the automaton builder against the sum over all labellings, on sequences short enough to
    enumerate (the reference checks the loop-free one against TensorFlow's loss with ctc_merge_repeated=False,
    tests/test_TFNativeOp.py:1815-1826; torch's loss has no such switch)."""
    announce("reference op GetCtcFsaFastBwOp, label_loop", label_loop)
    make_fsa, baum_welch = _op("GetCtcFsaFastBwOp"), _op("FastBaumWelchOp")
    targets = numpy.array([[0, 1, 1], [1, 1, 0], [2, 0, 0]], dtype=numpy.int32)
    target_lens = numpy.array([3, 2, 1], dtype=numpy.int32)
    n_classes, blank = 4, 3
    lens = numpy.array([6, 5, 4])
    n_time, n_batch = 6, 3
    logits = numpy.random.RandomState(11).normal(size=(n_time, n_batch, n_classes)).astype(numpy.float32)
    log_probs = torch.log_softmax(torch.tensor(logits, dtype=torch.float64), dim=2).numpy()
    n_edges = n_batch * (5 * (targets.shape[1] - 1) + 10)
    weights = torch.zeros((n_edges,), device="cuda:0")
    edges, start_end = make_fsa(_dev(targets), _dev(target_lens), blank, weights, int(label_loop))
    n_states = int(_host(start_end)[1].max()) + 1
    index = (numpy.arange(n_time)[:, None] < lens[None, :]).astype(numpy.float32)
    fwdbwd, scores = baum_welch(_dev((-log_probs).astype(numpy.float32)), edges, weights, start_end, _dev(index), n_states)
    scores = _host(scores)
    for b in range(n_batch):
        want = _paths_by_enumeration(log_probs[: lens[b], b], targets[b, : target_lens[b]], blank, label_loop)
        numpy.testing.assert_allclose(scores[: lens[b], b], want, rtol=2e-5)


@needs("GetCtcFsaFastBwPackedOp", "FastBaumWelchOp", "FastBaumWelchPackedOp")
@pytest.mark.parametrize("case", [0, 1, 4, 7])
def test_packed_ctc_automaton_and_packed_baum_welch(case):
    targets, target_lens, logits, lens = _ctc_inputs(*CTC_TARGETS[case])
    announce("reference ops GetCtcFsaFastBwPackedOp + FastBaumWelchPackedOp", targets.shape, target_lens.tolist())
    make_fsa, baum_welch, baum_welch_packed = _op("GetCtcFsaFastBwPackedOp"), _op("FastBaumWelchOp"), _op("FastBaumWelchPackedOp")
    n_batch = targets.shape[0]
    n_time, _, n_classes = logits.shape
    blank = n_classes - 1
    offsets = numpy.concatenate([[0], numpy.cumsum(5 * target_lens + 5)]).astype(numpy.int32)  # returnn/native_op.py:5728-5730
    n_edges = int(offsets[-1]) + 3  # (a bound with some filler behind the last sequence's slice)
    weights = torch.zeros((n_edges,), device="cuda:0")
    edges, start_end = make_fsa(_dev(targets), _dev(target_lens), _dev(offsets), blank, weights, 1)
    assert tuple(edges.shape) == (4, n_edges) and tuple(start_end.shape) == (2, n_batch)
    n_states = int(_host(start_end)[1].max()) + 1
    index = (numpy.arange(n_time)[:, None] < lens[None, :]).astype(numpy.float32)
    am = -torch.log_softmax(torch.tensor(logits, dtype=torch.float64), dim=2).numpy().astype(numpy.float32)
    fwdbwd, scores = baum_welch(_dev(am), edges, weights, start_end, _dev(index), n_states)
    fwdbwd, scores = _host(fwdbwd), _host(scores)
    _check_against_ctc(fwdbwd, scores, logits, lens, targets, target_lens, blank)
    # the same sequences without padding: frames of sequence b at seq_starts[b] ... of one flat array
    seq_starts = numpy.concatenate([[0], numpy.cumsum(lens)[:-1]]).astype(numpy.int32)
    packed = numpy.concatenate([am[: lens[b], b] for b in range(n_batch)], axis=0)
    p_fwdbwd, p_scores = baum_welch_packed(_dev(packed), edges, weights, start_end, _dev(index), _dev(seq_starts), n_states)
    p_fwdbwd, p_scores = _host(p_fwdbwd), _host(p_scores)
    assert p_fwdbwd.shape == packed.shape and p_scores.shape == scores.shape
    for b in range(n_batch):
        numpy.testing.assert_allclose(p_scores[: lens[b], b], scores[: lens[b], b], rtol=1e-5)
        got = numpy.exp(-p_fwdbwd[seq_starts[b] : seq_starts[b] + lens[b]].astype(numpy.float64))
        numpy.testing.assert_allclose(got, numpy.exp(-fwdbwd[: lens[b], b].astype(numpy.float64)), rtol=1e-3, atol=1e-6)
