"""Plain numpy forward-backward and Viterbi over a batch automaton given as edge lists (from, to, label, sequence): the
textbook recursions, written for the tests that run the reference's FastBaumWelchOp / FastViterbiOp after this package's op
loader has compiled them.  Pinned by the known answers of tests/golden/ref_op_cases.npz (tests/test_ref_op_cases.py)."""

from __future__ import annotations

import numpy


def _logaddexp_neg(a, b):
    """-log(exp(-a) + exp(-b)) for scores in -log space (inf = impossible)."""
    return -numpy.logaddexp(-a, -b)


def baum_welch(am_scores, index, edges, weights, start_end_states, n_states):
    """
    :param am_scores: [T,B,D] in -log space
    :param index: [T,B] 1 for frames inside the sequence
    :return: fwdbwd [T,B,D] in -log space (normalised per frame: exp(-fwdbwd) sums to 1 over D), score [T,B] = -log of the
        total path probability (the same in every frame of a sequence)
    """
    T, B, D = am_scores.shape
    E = edges.shape[1]
    inf = numpy.inf
    fwd = numpy.full((T + 1, n_states), inf)
    bwd = numpy.full((T + 1, n_states), inf)
    lens = index.sum(axis=0).astype(int)
    for b in range(B):
        fwd[0, start_end_states[0, b]] = 0.0
    for t in range(T):
        for e in range(E):
            src, dst, label, seq = edges[:, e]
            if t < lens[seq] and fwd[t, src] < inf:
                fwd[t + 1, dst] = _logaddexp_neg(fwd[t + 1, dst], fwd[t, src] + weights[e] + am_scores[t, seq, label])
    for b in range(B):
        bwd[lens[b], start_end_states[1, b]] = 0.0
    for t in range(T - 1, -1, -1):
        for e in range(E):
            src, dst, label, seq = edges[:, e]
            if t < lens[seq] and bwd[t + 1, dst] < inf:
                bwd[t, src] = _logaddexp_neg(bwd[t, src], bwd[t + 1, dst] + weights[e] + am_scores[t, seq, label])
    out = numpy.full((T, B, D), inf)
    for t in range(T):
        for e in range(E):
            src, dst, label, seq = edges[:, e]
            if t < lens[seq]:
                v = fwd[t, src] + weights[e] + am_scores[t, seq, label] + bwd[t + 1, dst]
                out[t, seq, label] = _logaddexp_neg(out[t, seq, label], v)
    score = -numpy.logaddexp.reduce(-out, axis=2)  # [T,B]
    return out - score[:, :, None], score


def viterbi(am_scores, am_seq_len, edges, weights, start_end_states, n_states):
    """
    :param am_scores: [T,B,D] in +log space
    :return: alignment [T,B] (label per frame on the best path), score [B] in +log space
    """
    T, B, D = am_scores.shape
    E = edges.shape[1]
    ninf = -numpy.inf
    best = numpy.full((T + 1, n_states), ninf)
    back = numpy.full((T + 1, n_states), -1, dtype=int)
    for b in range(B):
        best[0, start_end_states[0, b]] = 0.0
    for t in range(T):
        for e in range(E):
            src, dst, label, seq = edges[:, e]
            if t < am_seq_len[seq] and best[t, src] > ninf:
                v = best[t, src] + weights[e] + am_scores[t, seq, label]
                if v > best[t + 1, dst]:
                    best[t + 1, dst], back[t + 1, dst] = v, e
    align = numpy.zeros((T, B), dtype=numpy.int32)
    score = numpy.zeros((B,))
    for b in range(B):
        state = start_end_states[1, b]
        score[b] = best[am_seq_len[b], state]
        for t in range(am_seq_len[b], 0, -1):
            e = back[t, state]
            align[t - 1, b] = edges[2, e]
            state = edges[0, e]
    return align, score
