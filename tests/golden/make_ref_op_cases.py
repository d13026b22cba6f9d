"""
Writes ``ref_op_cases.npz``: inputs and expected results of seven of the reference's other native ops, for the test
that runs those ops on the GPU after the op loader of this package has compiled them.  Run from the repository root:
``python tests/golden/make_ref_op_cases.py``.  Needs nothing from the reference tree.

Everything expected here is DATA that the reference's own tests hold, retyped from tests/test_torch_native_op.py:

* ``test_fast_bw_uniform`` (:95-160): a left-to-right automaton over 5 labels (edge ``i -> i+1`` and loop ``i+1 -> i+1``,
  both emitting label ``i``), 7 frames, 3 sequences, uniform scores ``-log(1/5)``: the score is 8.55801582 in every frame
  and sequence, and ``exp(-fwdbwd)`` is the 7 x 5 table ``ref_align``;
* ``test_fast_viterbi`` (:582-631): the same automaton, scores = log of the 5 x 5 identity stretched to 7 frames by
  linear interpolation: score -1.6218603, alignment ``[0, 1, 1, 2, 3, 3, 4]``;
* ``test_edit_distance`` (:689-754): eight explicit pairs with distances 1, 1, 2, 1, 1, 1, 0, 2 inside a batch of 15
  drawn from ``RandomState(42)``, and ``test_edit_distance_ref_np_b1`` (:905-912): seven pairs with distances
  1, 1, 2, 1, 1, 2, 1;
* ``test_optimal_completion_edit_distance`` (:922-976): seven explicit pairs with results 1, 0, 1, 1, 1, 0, 0 inside
  another batch of 15;
* ``test_optimal_completion_edit_distance_per_successor`` (:1036-1135): seven explicit pairs with results 1, 0, 1, 1, 1, 0, 0
  (the sixth other than above: labels stay below the 10 classes) for the successor that is the prefix's own last label,
  inside a batch of 15; the op is given the prefixes without their last label and returns one result per successor label;
* ``test_next_edit_distance_row`` (:1137-1276) and ``test_next_edit_distance_row_optimal_completion`` (:1278-1365): the
  batches of ``test_edit_distance`` and ``test_optimal_completion_edit_distance`` again, computed one row of the
  dynamic programme per op call;
* ``test_next_edit_distance_reduce_optimal_completion`` (:1367-1400): a batch of 15 with prefixes of full length 7, one
  result per successor label (no numbers held: every entry is left to the reference's naive routine).

Where the reference's test leaves an entry of the batch to its own numpy routine (the random rest), the expected number
is computed here by the textbook dynamic programme below; ``*_held`` marks the entries the reference holds as numbers,
and the textbook routine must reproduce every one of those before anything is written.
"""

from __future__ import annotations

import os

import numpy


def levenshtein(a, b) -> int:
    """Insertions, deletions and substitutions of weight 1 (Wagner-Fischer)."""
    prev = list(range(len(b) + 1))
    for i in range(1, len(a) + 1):
        cur = [i] + [0] * len(b)
        for j in range(1, len(b) + 1):
            cur[j] = min(prev[j] + 1, cur[j - 1] + 1, prev[j - 1] + (0 if a[i - 1] == b[j - 1] else 1))
        prev = cur
    return prev[len(b)]


def optimal_completion(a, b) -> int:
    """The smallest distance between ``a`` and any prefix of ``b``."""
    return min(levenshtein(a, b[:k]) for k in range(len(b) + 1))


def left_to_right_fsa(n_classes: int, n_batch: int):
    """Edges (from, to, label, sequence), weights and (start, end) states of one automaton repeated per sequence, states
    numbered consecutively over the batch (the layout of returnn/util/fsa.py:1092-1137)."""
    single = []
    for i in range(n_classes):
        single.append((i, i + 1, i))
        single.append((i + 1, i + 1, i))
    n_states = n_classes + 1
    edges = numpy.zeros((4, len(single) * n_batch), dtype=numpy.int32)
    for b in range(n_batch):
        for e, (src, dst, label) in enumerate(single):
            edges[:, b * len(single) + e] = (src + b * n_states, dst + b * n_states, label, b)
    weights = numpy.zeros((edges.shape[1],), dtype=numpy.float32)
    start_end = numpy.array([[b * n_states for b in range(n_batch)], [n_states - 1 + b * n_states for b in range(n_batch)]], dtype=numpy.int32)
    return edges, weights, start_end, n_states * n_batch


def fast_bw_uniform():
    n_batch, seq_len, n_classes = 3, 7, 5
    edges, weights, start_end, n_states = left_to_right_fsa(n_classes, n_batch)
    am = -numpy.log(numpy.ones((seq_len, n_batch, n_classes), dtype=numpy.float32) * numpy.float32(1.0 / n_classes))
    ref_align = numpy.array(
        [
            [1.0, 0.0, 0.0, 0.0, 0.0],
            [0.33333316, 0.66666663, 0.0, 0.0, 0.0],
            [0.06666669, 0.53333354, 0.40000018, 0.0, 0.0],
            [0.0, 0.20000014, 0.60000014, 0.19999999, 0.0],
            [0.0, 0.0, 0.39999962, 0.53333312, 0.06666663],
            [0.0, 0.0, 0.0, 0.66666633, 0.33333316],
            [0.0, 0.0, 0.0, 0.0, 0.99999982],
        ],
        dtype=numpy.float32,
    )
    return {
        "bw_am_scores": am.astype(numpy.float32), "bw_edges": edges, "bw_weights": weights, "bw_start_end_states": start_end,
        "bw_index": numpy.ones((seq_len, n_batch), dtype=numpy.float32), "bw_n_states": numpy.int32(n_states),
        "bw_score": numpy.float32(8.55801582), "bw_align": numpy.tile(ref_align[:, None, :], (1, n_batch, 1)),
    }  # fmt: skip


def fast_viterbi():
    import scipy.ndimage

    n_batch, seq_len, n_classes = 3, 7, 5
    edges, weights, start_end, n_states = left_to_right_fsa(n_classes, n_batch)
    am = numpy.eye(n_classes, n_classes, dtype="float32")
    am = scipy.ndimage.zoom(am, zoom=(float(seq_len) / n_classes, 1), order=1, prefilter=False)
    assert am.shape == (seq_len, n_classes)
    am = am[:, None] + numpy.zeros((seq_len, n_batch, n_classes), dtype="float32")
    with numpy.errstate(divide="ignore"):
        am = numpy.log(am)  # +log space; -inf where the stretched identity is 0
    return {
        "vit_am_scores": am.astype(numpy.float32), "vit_am_seq_len": numpy.full((n_batch,), seq_len, dtype=numpy.int32),
        "vit_edges": edges, "vit_weights": weights, "vit_start_end_states": start_end, "vit_n_states": numpy.int32(n_states),
        "vit_score": numpy.float32(-1.6218603), "vit_alignment": numpy.array([0, 1, 1, 2, 3, 3, 4], dtype=numpy.int32),
    }  # fmt: skip


def _batch(rnd, n_batch, n_a_max_len, n_b_max_len, explicit, fn):
    num_classes = 10
    a = rnd.randint(0, num_classes, size=(n_batch, n_a_max_len), dtype="int32")
    b = rnd.randint(0, num_classes, size=(n_batch, n_b_max_len), dtype="int32")
    a_len = rnd.randint(1, n_a_max_len + 1, size=(n_batch,), dtype="int32")
    b_len = rnd.randint(1, n_b_max_len + 1, size=(n_batch,), dtype="int32")
    held = numpy.zeros((n_batch,), dtype=bool)
    expected = numpy.zeros((n_batch,), dtype=numpy.int32)
    for i, (sa, sb, la, lb, want) in enumerate(explicit):
        a[i, : len(sa)] = sa
        b[i, : len(sb)] = sb
        a_len[i], b_len[i] = la, lb
        held[i], expected[i] = True, want
    for i in range(n_batch):
        got = fn(list(a[i, : a_len[i]]), list(b[i, : b_len[i]]))
        if held[i]:
            assert got == expected[i], ("the textbook routine disagrees with a number the reference holds", i, got, expected[i])
        expected[i] = got
    return a, a_len, b, b_len, expected, held


def edit_distance():
    explicit = [
        ([1], [], 1, 0, 1),
        ([1, 2], [1], 2, 1, 1),
        ([1, 2], [3], 2, 1, 2),
        ([1, 2, 3, 4], [1, 2, 4, 4], 4, 4, 1),
        ([1, 2, 3, 3, 4, 5], [1, 2, 3, 4, 5], 6, 5, 1),
        ([1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 4, 5, 6], 6, 7, 1),
        ([2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 11], [2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 11], 11, 11, 0),
        ([2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 0, 0, 0], [2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 0], 13, 11, 2),
    ]
    a, a_len, b, b_len, expected, held = _batch(numpy.random.RandomState(42), 15, 13, 11, explicit, levenshtein)
    out = {"ed_a": a, "ed_a_len": a_len, "ed_b": b, "ed_b_len": b_len, "ed_expected": expected, "ed_held": held}
    pairs = [([1], [], 1), ([1, 2], [1], 1), ([2, 2], [1], 2), ([2, 1], [1], 1), ([2, 1], [1, 1], 1), ([2, 1], [1, 1, 1], 2), ([2, 1], [2, 1, 1], 1)]
    pa = numpy.zeros((len(pairs), 2), dtype=numpy.int32)
    pb = numpy.zeros((len(pairs), 3), dtype=numpy.int32)
    pal, pbl, pe = (numpy.zeros((len(pairs),), dtype=numpy.int32) for _ in range(3))
    for i, (sa, sb, want) in enumerate(pairs):
        assert levenshtein(sa, sb) == want
        pa[i, : len(sa)], pb[i, : len(sb)] = sa, sb
        pal[i], pbl[i], pe[i] = len(sa), len(sb), want
    out.update({"ed1_a": pa, "ed1_a_len": pal, "ed1_b": pb, "ed1_b_len": pbl, "ed1_expected": pe})
    return out


def optimal_completion_edit_distance():
    explicit = [
        ([1], [], 1, 0, 1),
        ([1], [1, 2], 1, 2, 0),
        ([1], [3, 1], 1, 2, 1),
        ([1, 2, 3, 4], [1, 2, 4, 4], 4, 4, 1),
        ([1, 2, 3, 4, 5], [1, 2, 3, 3, 4, 5], 5, 6, 1),
        ([2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 11], [2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 11], 11, 11, 0),
        ([2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 0], [2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 0, 0, 0], 11, 13, 0),
    ]
    a, a_len, b, b_len, expected, held = _batch(numpy.random.RandomState(42), 15, 11, 13, explicit, optimal_completion)
    return {"oc_a": a, "oc_a_len": a_len, "oc_b": b, "oc_b_len": b_len, "oc_expected": expected, "oc_held": held}


def per_successor():
    """OptimalCompletionEditDistancePerSuccessorOp: ``expected[i, j]`` = smallest distance between the prefix of sequence i
    without its last label, followed by label j, and any prefix of b."""
    num_classes = 10
    explicit = [
        ([1], [], 1, 0, 1),
        ([1], [1, 2], 1, 2, 0),
        ([1], [3, 1], 1, 2, 1),
        ([1, 2, 3, 4], [1, 2, 4, 4], 4, 4, 1),
        ([1, 2, 3, 4, 5], [1, 2, 3, 3, 4, 5], 5, 6, 1),
        ([2, 2, 4, 4, 6, 6, 8, 8, 9, 1, 3], [2, 2, 4, 4, 6, 6, 8, 8, 9, 1, 3], 11, 11, 0),
        ([2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 0], [2, 2, 4, 4, 6, 6, 8, 8, 9, 10, 0, 0, 0], 11, 13, 0),
    ]
    a, a_len, b, b_len, whole, held = _batch(numpy.random.RandomState(42), 15, 11, 13, explicit, optimal_completion)
    expected = numpy.zeros((a.shape[0], num_classes), dtype=numpy.int32)
    for i in range(a.shape[0]):
        for j in range(num_classes):
            expected[i, j] = optimal_completion(list(a[i, : a_len[i] - 1]) + [j], list(b[i, : b_len[i]]))
        last = int(a[i, a_len[i] - 1])
        assert 0 <= last < num_classes and expected[i, last] == whole[i]  # the held numbers sit in this column
    return {"ps_a": a, "ps_a_len": a_len, "ps_b": b, "ps_b_len": b_len, "ps_expected": expected, "ps_whole": whole, "ps_held": held,
            "ps_num_classes": numpy.int32(num_classes)}  # fmt: skip


def next_reduce():
    """NextEditDistanceReduceOp after all of a has been consumed row by row: ``expected[i, j]`` = smallest distance between
    a[i] followed by label j and any prefix of b[i]."""
    rnd = numpy.random.RandomState(42)
    n_batch, n_a, n_b, num_classes = 15, 7, 13, 10
    a = rnd.randint(0, num_classes, size=(n_batch, n_a), dtype="int32")
    b = rnd.randint(0, num_classes, size=(n_batch, n_b), dtype="int32")
    a_len = numpy.array([n_a] * n_batch, dtype="int32")
    b_len = rnd.randint(1, n_b + 1, size=(n_batch,), dtype="int32")
    expected = numpy.zeros((n_batch, num_classes), dtype=numpy.int32)
    for i in range(n_batch):
        for j in range(num_classes):
            expected[i, j] = optimal_completion(list(a[i]) + [j], list(b[i, : b_len[i]]))
    return {"nr_a": a, "nr_a_len": a_len, "nr_b": b, "nr_b_len": b_len, "nr_expected": expected, "nr_num_classes": numpy.int32(num_classes)}


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    out = {}
    for part in (fast_bw_uniform(), fast_viterbi(), edit_distance(), optimal_completion_edit_distance(), per_successor(), next_reduce()):
        out.update(part)
    numpy.savez_compressed(os.path.join(here, "ref_op_cases.npz"), **out)
    print("wrote ref_op_cases.npz:", ", ".join(sorted(out)))


if __name__ == "__main__":
    main()
