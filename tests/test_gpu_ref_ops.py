"""
Seven of the reference's other native ops (FastBaumWelchOp, FastViterbiOp, EditDistanceOp,
OptimalCompletionEditDistanceOp, OptimalCompletionEditDistancePerSuccessorOp, NextEditDistanceRowOp,
NextEditDistanceReduceOp), compiled for gfx950 by this package's op loader from the reference's own op sources,
run on the GPU against the numbers the reference's tests hold (tests/golden/ref_op_cases.npz) and, beyond those, against
the plain numpy recursions that the same numbers pin (tests/test_ref_op_cases.py).

The shared objects are built where the reference tree is (``python tests/build_ref_ops.py``, also part of the build
step) into ``tests/_built_ref_ops/``; here they are only loaded.  This checks the loader -- dialect header, generated entry
point, argument conversion, device allocation callbacks -- on code that was not written for it.
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
CASES = os.path.join(ROOT, "tests", "golden", "ref_op_cases.npz")

needs_ops = pytest.mark.skipif(
    not os.path.exists(os.path.join(OPS_DIR, "ops.json")),
    reason="tests/_built_ref_ops is not built (python tests/build_ref_ops.py, where the reference tree is)",
)


def _op(name):
    table = json.load(open(os.path.join(OPS_DIR, "ops.json")))
    return op_loader.CompiledOp.from_shared_object(name, table[name]["in_info"], table[name]["out_info"], os.path.join(OPS_DIR, name + ".so"))


def _dev(a):
    return torch.from_numpy(numpy.ascontiguousarray(a)).to("cuda:0")


@needs_ops
def test_fast_baum_welch_known_answer_and_random():
    announce("reference op FastBaumWelchOp")
    c = dict(numpy.load(CASES))
    op = _op("FastBaumWelchOp")
    fwdbwd, score = op(_dev(c["bw_am_scores"]), _dev(c["bw_edges"]), _dev(c["bw_weights"]), _dev(c["bw_start_end_states"]),
                       _dev(c["bw_index"]), int(c["bw_n_states"]))  # fmt: skip
    torch.cuda.synchronize()
    fwdbwd, score = fwdbwd.cpu().numpy(), score.cpu().numpy()
    assert score.shape == (7, 3) and fwdbwd.shape == (7, 3, 5)
    numpy.testing.assert_allclose(score, float(c["bw_score"]), rtol=1e-5)  # tolerance of the reference's test
    numpy.testing.assert_allclose(numpy.exp(-fwdbwd), c["bw_align"], rtol=1e-5, atol=1e-6)
    # random scores and ragged lengths, against the numpy recursion (the case of the reference's test_FastBaumWelch
    # with another automaton; its own check is against its numpy routine too)
    rng = numpy.random.RandomState(42)
    T, B, D = 9, 4, 5
    am = rng.normal(size=(T, B, D)).astype(numpy.float32)
    lens = numpy.array([9, 7, 6, 9])
    index = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_ref_op_cases", os.path.join(ROOT, "tests", "golden", "make_ref_op_cases.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    edges, weights, start_end, n_states = mod.left_to_right_fsa(D, B)
    weights = rng.uniform(0.0, 0.5, size=weights.shape).astype(numpy.float32)
    fwdbwd, score = op(_dev(am), _dev(edges), _dev(weights), _dev(start_end), _dev(index), int(n_states))
    torch.cuda.synchronize()
    want_fb, want_score = _fsa_numpy.baum_welch(am.astype(numpy.float64), index, edges, weights.astype(numpy.float64), start_end, n_states)
    inside = index.astype(bool)
    numpy.testing.assert_allclose(score.cpu().numpy()[inside], want_score[inside], rtol=1e-4)
    got = numpy.exp(-fwdbwd.cpu().numpy().astype(numpy.float64))
    numpy.testing.assert_allclose(got[inside], numpy.exp(-want_fb)[inside], rtol=1e-3, atol=1e-5)


@needs_ops
def test_fast_viterbi_known_answer():
    announce("reference op FastViterbiOp")
    c = dict(numpy.load(CASES))
    op = _op("FastViterbiOp")
    align, score = op(_dev(c["vit_am_scores"]), _dev(c["vit_am_seq_len"]), _dev(c["vit_edges"]), _dev(c["vit_weights"]),
                      _dev(c["vit_start_end_states"]), int(c["vit_n_states"]), 0)  # fmt: skip
    torch.cuda.synchronize()
    align, score = align.cpu().numpy(), score.cpu().numpy()
    assert align.shape == (7, 3) and score.shape == (3,)
    numpy.testing.assert_allclose(score, float(c["vit_score"]), rtol=1e-5)
    for b in range(3):
        assert align[:, b].tolist() == c["vit_alignment"].tolist()


@needs_ops
@pytest.mark.parametrize("name,prefix", [("EditDistanceOp", "ed"), ("OptimalCompletionEditDistanceOp", "oc")])
def test_edit_distance_known_answers(name, prefix):
    announce("reference op", name)
    c = dict(numpy.load(CASES))
    op = _op(name)
    a, a_len, b, b_len, want = (c["%s_%s" % (prefix, k)] for k in ("a", "a_len", "b", "b_len", "expected"))
    (got,) = op(_dev(a), _dev(a_len), _dev(b), _dev(b_len))
    torch.cuda.synchronize()
    assert got.cpu().numpy().tolist() == want.tolist()
    # one pair at a time, cut to its own lengths, as the reference's test does
    for i in range(a.shape[0]):
        (one,) = op(_dev(a[i : i + 1, : a_len[i]]), _dev(a_len[i : i + 1]), _dev(b[i : i + 1, : b_len[i]]), _dev(b_len[i : i + 1]))
        assert int(one.cpu()[0]) == int(want[i]), i
    if prefix == "ed":
        (swapped,) = op(_dev(b), _dev(b_len), _dev(a), _dev(a_len))  # the distance is symmetric
        assert swapped.cpu().numpy().tolist() == want.tolist()
        (got1,) = op(_dev(c["ed1_a"]), _dev(c["ed1_a_len"]), _dev(c["ed1_b"]), _dev(c["ed1_b_len"]))
        assert got1.cpu().numpy().tolist() == c["ed1_expected"].tolist()


@needs_ops
def test_optimal_completion_per_successor_known_answers():
    """tests/test_torch_native_op.py:1036-1135: the op gets every prefix without its last label and answers for all ten
    successor labels; the numbers the reference holds are those of the prefix's own last label."""
    announce("reference op OptimalCompletionEditDistancePerSuccessorOp")
    c = dict(numpy.load(CASES))
    op = _op("OptimalCompletionEditDistancePerSuccessorOp")
    a, a_len, b, b_len = c["ps_a"], c["ps_a_len"], c["ps_b"], c["ps_b_len"]
    n_labels = int(c["ps_num_classes"])
    (got,) = op(_dev(a), _dev(a_len - 1), _dev(b), _dev(b_len), _dev(numpy.arange(n_labels, dtype=numpy.int32)))
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert got.shape == (a.shape[0], n_labels)
    assert got.tolist() == c["ps_expected"].tolist()
    for i in range(a.shape[0]):
        assert int(got[i, a[i, a_len[i] - 1]]) == int(c["ps_whole"][i])
    assert c["ps_held"].sum() == 7 and c["ps_whole"][c["ps_held"]].tolist() == [1, 0, 1, 1, 1, 0, 0]


def _rows(op, a, a_len, b, b_len):
    """The dynamic programme one row per op call (the protocol of returnn/torch/util/native_op.py:1129-1160): the row
    starts as 0..b_time for every sequence; call i hands over label i of every sequence and whether it has ended."""
    n_batch, time1 = a.shape
    row = _dev(numpy.tile(numpy.arange(b.shape[1] + 1, dtype=numpy.int32)[None], (n_batch, 1)))
    bd, bl = _dev(b), _dev(b_len)
    for i in range(time1):
        ended = (i >= a_len).astype(numpy.int32)
        (row,) = op(row, _dev(a[:, i]), _dev(numpy.full((n_batch,), i, dtype=numpy.int32)), _dev(ended), bd, bl)
    return row


@needs_ops
def test_next_edit_distance_row_known_answers():
    """tests/test_torch_native_op.py:1137-1365: the batches of the two edit-distance tests, row by row: the last entry of
    the final row is the edit distance (whole batch, pair by pair cut to its lengths, and with the roles swapped), its
    minimum the optimal-completion distance."""
    announce("reference op NextEditDistanceRowOp")
    c = dict(numpy.load(CASES))
    op = _op("NextEditDistanceRowOp")
    a, a_len, b, b_len, want = (c["ed_%s" % k] for k in ("a", "a_len", "b", "b_len", "expected"))
    assert c["ed_held"].sum() == 8 and want[c["ed_held"]].tolist() == [1, 1, 2, 1, 1, 1, 0, 2]
    assert _rows(op, a, a_len, b, b_len)[:, -1].cpu().numpy().tolist() == want.tolist()
    assert _rows(op, b, b_len, a, a_len)[:, -1].cpu().numpy().tolist() == want.tolist()
    for i in range(a.shape[0]):
        ai, bi = a[i : i + 1, : a_len[i]], b[i : i + 1, : b_len[i]]
        assert int(_rows(op, ai, a_len[i : i + 1], bi, b_len[i : i + 1])[0, -1].cpu()) == int(want[i]), i
        assert int(_rows(op, bi, b_len[i : i + 1], ai, a_len[i : i + 1])[0, -1].cpu()) == int(want[i]), i
    a, a_len, b, b_len, want = (c["oc_%s" % k] for k in ("a", "a_len", "b", "b_len", "expected"))
    assert want[c["oc_held"]].tolist() == [1, 0, 1, 1, 1, 0, 0]
    assert _rows(op, a, a_len, b, b_len).min(dim=1).values.cpu().numpy().tolist() == want.tolist()


@needs_ops
def test_next_edit_distance_reduce_answers():
    """tests/test_torch_native_op.py:1367-1400 (and returnn/torch/util/native_op.py:1188-1217 for the protocol): all of a
    row by row, then one call that answers for every successor label."""
    announce("reference op NextEditDistanceReduceOp")
    c = dict(numpy.load(CASES))
    row_op, op = _op("NextEditDistanceRowOp"), _op("NextEditDistanceReduceOp")
    a, a_len, b, b_len = c["nr_a"], c["nr_a_len"], c["nr_b"], c["nr_b_len"]
    n_labels = int(c["nr_num_classes"])
    last_row = _rows(row_op, a, a_len, b, b_len)
    n_batch = a.shape[0]
    (got,) = op(last_row, _dev(numpy.arange(n_labels, dtype=numpy.int32)[None]), _dev(numpy.full((n_batch,), a.shape[1], dtype=numpy.int32)),
                _dev((a_len != a.shape[1]).astype(numpy.int32)), _dev(b), _dev(b_len), 1, -1)  # fmt: skip
    torch.cuda.synchronize()
    assert got.cpu().numpy().tolist() == c["nr_expected"].tolist()
