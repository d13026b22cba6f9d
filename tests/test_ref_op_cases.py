"""The known answers of tests/golden/ref_op_cases.npz against plain numpy recursions (no GPU, no reference tree): the file
is what its script writes, the textbook routines reproduce every number the reference's tests hold, and so they can
stand in for cases the reference's tests leave to their own numpy code."""

from __future__ import annotations

import importlib.util
import os

import numpy

import _fsa_numpy

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _script():
    spec = importlib.util.spec_from_file_location("make_ref_op_cases", os.path.join(GOLDEN, "make_ref_op_cases.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _cases():
    return dict(numpy.load(os.path.join(GOLDEN, "ref_op_cases.npz")))


def test_file_is_what_the_script_writes():
    mod, stored = _script(), _cases()
    fresh = {}
    for part in (mod.fast_bw_uniform(), mod.fast_viterbi(), mod.edit_distance(), mod.optimal_completion_edit_distance(),
                 mod.per_successor(), mod.next_reduce()):
        fresh.update(part)
    assert sorted(fresh) == sorted(stored)
    for k in fresh:
        numpy.testing.assert_array_equal(numpy.asarray(fresh[k]), stored[k], err_msg=k)


def test_baum_welch_known_answer():
    c = _cases()
    fwdbwd, score = _fsa_numpy.baum_welch(c["bw_am_scores"].astype(numpy.float64), c["bw_index"], c["bw_edges"], c["bw_weights"],
                                          c["bw_start_end_states"], int(c["bw_n_states"]))  # fmt: skip
    numpy.testing.assert_allclose(score, float(c["bw_score"]), rtol=1e-6)
    numpy.testing.assert_allclose(numpy.exp(-fwdbwd), c["bw_align"], rtol=1e-5, atol=1e-6)
    # closed form: 5 labels in order over 7 frames, each at least once: choose(6, 4) = 15 paths of probability 5^-7 each
    numpy.testing.assert_allclose(float(c["bw_score"]), 7 * numpy.log(5.0) - numpy.log(15.0), rtol=1e-6)


def test_viterbi_known_answer():
    c = _cases()
    align, score = _fsa_numpy.viterbi(c["vit_am_scores"].astype(numpy.float64), c["vit_am_seq_len"], c["vit_edges"], c["vit_weights"],
                                      c["vit_start_end_states"], int(c["vit_n_states"]))  # fmt: skip
    numpy.testing.assert_allclose(score, float(c["vit_score"]), rtol=1e-5)
    for b in range(align.shape[1]):
        assert align[:, b].tolist() == c["vit_alignment"].tolist()


def test_edit_distance_numbers():
    mod, c = _script(), _cases()
    assert c["ed_held"].sum() == 8 and c["ed_expected"][c["ed_held"]].tolist() == [1, 1, 2, 1, 1, 1, 0, 2]
    assert c["oc_held"].sum() == 7 and c["oc_expected"][c["oc_held"]].tolist() == [1, 0, 1, 1, 1, 0, 0]
    assert c["ed1_expected"].tolist() == [1, 1, 2, 1, 1, 2, 1]
    for i in range(len(c["ed_expected"])):
        a, b = list(c["ed_a"][i, : c["ed_a_len"][i]]), list(c["ed_b"][i, : c["ed_b_len"][i]])
        assert mod.levenshtein(a, b) == mod.levenshtein(b, a) == c["ed_expected"][i]  # symmetric, as the reference checks by swapping
        assert abs(len(a) - len(b)) <= c["ed_expected"][i] <= max(len(a), len(b))


def test_successor_tables():
    """The per-successor tables: the column of a prefix's own last label holds the whole prefix's number (seven of them
    held by the reference), and the row-by-row dynamic programme the GPU test drives gives the same numbers in numpy."""
    mod, c = _script(), _cases()
    assert c["ps_held"].sum() == 7 and c["ps_whole"][c["ps_held"]].tolist() == [1, 0, 1, 1, 1, 0, 0]
    for i in range(c["ps_a"].shape[0]):
        last = int(c["ps_a"][i, c["ps_a_len"][i] - 1])
        assert c["ps_expected"][i, last] == c["ps_whole"][i]

    def next_row(row, label, b):  # one row of Wagner-Fischer
        new = [row[0] + 1]
        for j in range(1, len(b) + 1):
            new.append(min(row[j] + 1, new[j - 1] + 1, row[j - 1] + (0 if label == b[j - 1] else 1)))
        return new

    for i in range(c["nr_a"].shape[0]):
        b = list(c["nr_b"][i, : c["nr_b_len"][i]])
        row = list(range(len(b) + 1))
        for label in c["nr_a"][i]:
            row = next_row(row, int(label), b)
        for j in range(int(c["nr_num_classes"])):
            assert min(next_row(row, j, b)) == c["nr_expected"][i, j]
