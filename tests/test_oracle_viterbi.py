"""Pins the best-path oracle (oracle/viterbi_oracle.c) without running the reference:
the reference's own test vector, brute force over all paths, hand-worked tie and no-path cases,
and the low-temperature limit of the full-sum oracle."""
import numpy as np
import pytest

from tests.helpers import golden
from tests.helpers import random_fsa


def viterbi_fixture():
    """test/fast_viterbi.py:9-35: B=1, T=5, F=2, two states, three edges, all weights 1."""
    from tests.helpers import reference_viterbi_fixture
    return reference_viterbi_fixture()[0]


def all_paths(am, edges, weights, start_end, seq_lens, b):
    """Every accepting path of sequence b as (score in float64, tuple of edge indices)."""
    L = int(seq_lens[b])
    E = edges.shape[1]
    out_edges = {}
    for e in range(E):
        if edges[3, e] == b:
            out_edges.setdefault(int(edges[0, e]), []).append(e)
    found = []
    stack = [(int(start_end[0, b]), 0, 0.0, ())]
    while stack:
        s, t, sc, path = stack.pop()
        if t == L:
            if s == int(start_end[1, b]):
                found.append((sc, path))
            continue
        for e in out_edges.get(s, []):
            stack.append((int(edges[1, e]), t + 1, sc + float(weights[e]) + float(am[t, b, edges[2, e]]), path + (e,)))
    return found


def test_reference_vector(oracle):
    """test/fast_viterbi.py:37-42 expects [0, 0, 1, 1, 1]; the score follows from the five factors."""
    align, scores = oracle.viterbi_oracle(*viterbi_fixture())
    assert align[:, 0].tolist() == golden("fast_viterbi")["expected"]["alignment"]
    assert scores[0] == pytest.approx(5.0 + np.log(0.9 * 0.9 * 0.6 * 0.9 * 0.9), rel=1e-6)


@pytest.mark.parametrize("seed", range(40))
def test_brute_force(oracle, seed):
    rng = np.random.default_rng(7000 + seed)
    B, F, T = 2, 4, 6
    am, edges, weights, start_end, seq_lens, n_states = random_fsa(rng, B, F, T=T)
    am = -am            # maximised scores
    align, scores = oracle.viterbi_oracle(am, edges, weights, start_end, seq_lens, n_states)
    for b in range(B):
        L = int(seq_lens[b])
        assert (align[L:, b] == 0).all()
        paths = all_paths(am, edges, weights, start_end, seq_lens, b)
        if not paths:
            assert scores[b] == -np.inf
            continue
        best = max(p[0] for p in paths)
        assert scores[b] == pytest.approx(best, abs=1e-4)
        # the emitted alignment must be that of a best path; with a clear winner it is unique
        winners = {tuple(int(edges[2, e]) for e in p[1]) for p in paths if p[0] > best - 1e-4}
        assert tuple(align[:L, b].tolist()) in winners


def test_tie_goes_to_the_earlier_edge(oracle):
    """core.cu:34-38: equal values keep the smaller edge index.  Two parallel edges with equal
    weight whose emissions have equal scores: the one listed first wins, whichever it is."""
    am = np.zeros((1, 1, 4), dtype=np.float32)
    for first, second in ((3, 2), (2, 3)):
        edges = np.array([[0, 1, first, 0], [0, 1, second, 0]], dtype=np.int32).T.copy()
        w = np.array([0.5, 0.5], dtype=np.float32)
        align, scores = oracle.viterbi_oracle(am, edges, w, np.array([[0], [1]], np.int32), np.array([1], np.int32), 2)
        assert align[:, 0].tolist() == [first]
        assert scores[0] == 0.5


def test_tie_between_source_states(oracle):
    """Diamond 0->{1,2}->3 with equal totals: state 3 keeps the back-pointer of the smaller edge
    index among (1->3, 2->3), and the path follows it."""
    am = np.zeros((2, 1, 6), dtype=np.float32)
    #            e0: 0->1 emits 1   e1: 0->2 emits 2   e2: 2->3 emits 4   e3: 1->3 emits 5
    edges = np.array([[0, 1, 1, 0], [0, 2, 2, 0], [2, 3, 4, 0], [1, 3, 5, 0]], dtype=np.int32).T.copy()
    w = np.zeros(4, dtype=np.float32)
    align, _ = oracle.viterbi_oracle(am, edges, w, np.array([[0], [3]], np.int32), np.array([2], np.int32), 4)
    assert align[:, 0].tolist() == [2, 4]          # through edge e2 (index 2 < 3), i.e. via state 2


def test_no_path_walk_back(oracle):
    """core.cu:160-171: a state without a back-pointer emits 0 and the walk stays there.  One edge
    0->1 (emission 5), two frames: the end state 1 is reached after one frame but not after two, so
    the score is -inf, frame 1 has no back-pointer (0) and frame 0 still finds the edge (5)."""
    am = np.zeros((2, 1, 6), dtype=np.float32)
    edges = np.array([[0, 1, 5, 0]], dtype=np.int32).T.copy()
    align, scores = oracle.viterbi_oracle(am, edges, np.zeros(1, np.float32), np.array([[0], [1]], np.int32),
                                          np.array([2], np.int32), 2)
    assert scores[0] == -np.inf
    assert align[:, 0].tolist() == [5, 0]


def test_zero_length(oracle):
    """seq_len 0: the score is read from frame 0 (0 at the start state, -inf elsewhere), no frame is aligned."""
    am = np.zeros((3, 2, 4), dtype=np.float32)
    edges = np.array([[0, 0, 1, 0], [1, 2, 2, 1]], dtype=np.int32).T.copy()
    se = np.array([[0, 1], [0, 2]], dtype=np.int32)
    align, scores = oracle.viterbi_oracle(am, edges, np.zeros(2, np.float32), se, np.array([0, 0], np.int32), 3)
    assert scores.tolist() == [0.0, -np.inf]
    assert (align == 0).all()


def test_padding_frames_are_zero_and_ignored(oracle):
    am, edges, weights, start_end, _, n = viterbi_fixture()
    align, scores = oracle.viterbi_oracle(am, edges, weights, start_end, np.array([4], np.int32), n)
    # best of the paths of length 4: forward edge in frame 1 -> 0.9 * 0.9 * 0.6 * 0.9
    assert align[:, 0].tolist() == [0, 0, 1, 1, 0]
    assert scores[0] == pytest.approx(4.0 + np.log(0.9 * 0.9 * 0.6 * 0.9), rel=1e-6)


def test_low_temperature_limit_of_full_sum(oracle):
    """-log sum_paths exp(-beta * cost) / beta -> min cost as beta grows: ties the best-path oracle
    to the full-sum oracle (which is pinned on its own) through an inequality with a known gap,
    0 <= min_cost - fbw(beta)/beta <= log(#paths)/beta."""
    rng = np.random.default_rng(99)
    T, B, F = 12, 2, 5
    # left-to-right chains with loops and skips
    frm, to, emis, seq = [], [], [], []
    off = 0
    for b in range(B):
        n = 5
        for s in range(n):
            frm += [off + s, off + s]; to += [off + s, off + s + 1]; emis += [int(rng.integers(0, F))] * 2; seq += [b, b]
            if s + 2 <= n:
                frm.append(off + s); to.append(off + s + 2); emis.append(int(rng.integers(0, F))); seq.append(b)
        off += n + 1
    edges = np.array([frm, to, emis, seq], dtype=np.int32)
    w = rng.uniform(0.1, 1.0, size=edges.shape[1]).astype(np.float32)
    se = np.array([[0, 6], [5, 11]], dtype=np.int32)
    lens = np.array([12, 9], dtype=np.int32)
    cost = rng.uniform(0.1, 3.0, size=(T, B, F)).astype(np.float32)
    _, scores = oracle.viterbi_oracle(-cost, edges, -w, se, lens, off)
    beta = 200.0
    _, loss = oracle.fbw_oracle(cost * beta, edges, w * beta, se, lens, off)
    for b in range(B):
        n_paths = len(all_paths(cost, edges, w, se, lens, b))
        gap = -scores[b] - loss[0, b] / beta
        assert -1e-4 <= gap <= np.log(n_paths) / beta + 1e-4


def test_workload_sized(oracle):
    """Score of the emitted alignment, re-accumulated along the path, equals the reported score."""
    from i6_native_ops_amd.fbw.workloads import make_workload
    wl = make_workload("monophone")
    am = -wl.am_scores
    align, scores = oracle.viterbi_oracle(am, wl.edges, -wl.weights, wl.start_end_states, wl.seq_lens, wl.n_states)
    assert np.isfinite(scores).all()
    for b in range(wl.B):
        L = int(wl.seq_lens[b])
        assert (align[L:, b] == 0).all()
        # every aligned emission belongs to an edge of the sequence
        emis_b = set(wl.edges[2, wl.edges[3] == b].tolist())
        assert set(align[:L, b].tolist()) <= emis_b
