"""Parity of the HIP path (through the C ABI of libi6fbw.so) with the CPU oracle.

Bar (fp32 path): loss relative error <= 1e-5, posterior absolute error <= 1e-4.
"""
import numpy as np
import pytest

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import brute_force, posterior, random_fsa, reference_fixture

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
POST_ATOL = 1e-4


def check_against_oracle(oracle, args, threads=1, bitwise=True):
    from i6_native_ops_amd import cabi
    from tests.gpu_util import run_cabi
    am, edges, weights, start_end, seq_lens, n_states = args
    want_out, want_loss = oracle.fbw_oracle(am, edges, weights, start_end, seq_lens, n_states, threads=threads)
    want_post = posterior(want_out)
    out, loss = run_cabi(*args, out_mode=cabi.OUT_NEG_LOG)
    np.testing.assert_allclose(loss, want_loss, rtol=LOSS_RTOL, atol=1e-6)
    assert (loss[want_loss == 0] == 0).all()
    np.testing.assert_allclose(posterior(out), want_post, rtol=0, atol=POST_ATOL)
    # holes are +inf in exactly the same places -- also where a posterior is below float's range: the reference adds in
    # log space (fbw_op.cu:115-134) and has a finite -log there -- and the finite values agree in the log domain too
    fin = np.isfinite(want_out)
    assert (np.isposinf(out) == ~fin).all()
    # (a -log above 69 is the difference of two numbers of the size of the loss, which is a float: half an ulp of it on top)
    np.testing.assert_allclose(out[fin], want_out[fin], rtol=2e-5, atol=2e-3 + 1.2e-7 * float(np.abs(want_loss).max()))
    prob, loss2 = run_cabi(*args, out_mode=cabi.OUT_PROB)
    # (the two modes add up the frame normaliser in different orders: per emission, and per edge where the -log output sums in
    # log space; the general path accumulates with atomics)
    np.testing.assert_allclose(loss2, loss, rtol=1e-6)
    if bitwise:      # the fast kernels sum in a fixed order: a second call gives the same bits
        prob_again, loss3 = run_cabi(*args, out_mode=cabi.OUT_PROB)
        np.testing.assert_array_equal(loss3, loss2)
        np.testing.assert_array_equal(prob_again, prob)
    np.testing.assert_allclose(prob, want_post, rtol=0, atol=POST_ATOL)
    assert (prob[np.isposinf(want_out)] == 0).all()
    return out, loss


@pytest.fixture(params=["single_stream", "overlapped"], autouse=True)
def schedule(request):
    """Every parity case runs under both schedules of i6fbw_run."""
    from i6_native_ops_amd import cabi
    cabi.set_overlap(0 if request.param == "single_stream" else 1)
    yield request.param
    cabi.set_overlap(-1)


@pytest.mark.parametrize("seq_len", [5, 4, 1, 0, 6, -3])
def test_reference_fixture(oracle, seq_len):
    out, loss = check_against_oracle(oracle, reference_fixture(seq_len))
    if seq_len == 5:   # closed form, test/fbw.py fixture
        np.testing.assert_allclose(loss[:, 0], 5 - np.log(0.73224), rtol=2e-6)
        np.testing.assert_allclose(posterior(out).sum(-1), 1.0, atol=1e-5)   # test/fbw.py:60-64


@pytest.mark.parametrize("seed", range(25))
def test_random_automata_brute_force(oracle, seed):
    rng = np.random.default_rng(100 + seed)
    args = random_fsa(rng, B=int(rng.integers(1, 5)), F=int(rng.integers(1, 6)), T=int(rng.integers(1, 8)))
    out, loss = check_against_oracle(oracle, args)
    want_loss, want_post = brute_force(*args)
    np.testing.assert_allclose(loss, want_loss, rtol=LOSS_RTOL, atol=1e-5)
    np.testing.assert_allclose(posterior(out), want_post, atol=POST_ATOL)


def test_tightly_constrained_alignment(oracle):
    """About one frame per state over more than a thousand states: the states that carry the posterior
    mass sit far from the frame minimum; the recursion keeps such sequences in double precision."""
    W = make_workload("cart", T=1150, B=3, F=400, n_labels=(366, 370))
    W.seq_lens[:] = [1150, 1120, 1135]
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=3)


@pytest.mark.parametrize("name,kw", [
    ("tiny", {}),
    ("tiny", dict(shuffle_edges=True)),
    ("monophone", dict(T=80, B=6, F=60)),
    ("monophone", {}),
    ("monophone", dict(shuffle_edges=True, seed=5)),
    ("cart", dict(T=120, B=4, F=500)),
    ("cart", dict(T=61, B=5, F=1024, n_labels=(5, 19))),       # the longest rows the row writer takes several frames at a time
    ("cart", dict(T=61, B=5, F=1025, n_labels=(5, 19))),       # one more float: frame by frame
    ("cart", dict(T=300, B=3, F=12001, shuffle_edges=True)),
    ("cart", dict(T=40, B=2, F=38000, n_labels=(8, 12))),     # the largest row images that fit into LDS
    ("ctc", dict(T=40, B=8, F=50)),
    ("ctc", dict(T=400, B=4, F=80, n_labels=(140, 190))),            # 560-940 edges, short rows: the row writer takes two frames at a time
    ("monophone", dict(T=420, B=6, F=264, n_labels=(130, 165))),     # 1000-1240 edges, short rows: one frame, eight edges per thread
    ("ctc", dict(T=200, B=16, F=5001, shuffle_edges=True)),
    ("cart", dict(T=60, B=44, F=300, n_labels=(5, 9))),      # the largest batch whose preparation holds the gather back itself: five workgroups per sequence, a unit each
    ("cart", dict(T=60, B=45, F=300, n_labels=(5, 9))),      # one more: a one-wave kernel does it
    ("ctc", dict(T=130, B=51, F=40, n_labels=(60, 80))),     # 5 B = 255 units in all, but 33 workgroups for the first XCD's 32 (this batch ran into the bound of its waits)
    ("cart", dict(T=60, B=64, F=300, n_labels=(5, 9))),      # a recursion workgroup on half of the compute units: started beside the preparation
    ("cart", dict(T=60, B=65, F=300, n_labels=(5, 9))),      # one more: started behind it
    ("cart", dict(T=60, B=128, F=300, n_labels=(5, 9))),     # one on every compute unit: gather and dense write must still find room
    ("ctc", dict(T=30, B=200, F=40)),          # 400 recursion workgroups: two per compute unit, started behind the preparation
    ("ctc", dict(T=30, B=256, F=40)),          # exactly two recursion workgroups on every compute unit
    ("ctc", dict(T=24, B=600, F=40)),          # more recursion workgroups than the device holds at once
    ("longform", dict(T=200, B=2, F=300)),
    ("longform", dict(T=1200, B=2, F=999, n_labels=(150, 200))),     # > 512 states: second size class
    ("longform", dict(T=4000, B=1, F=777, n_labels=(700, 800))),     # > 2048 states: third size class
])
def test_workloads_small(oracle, name, kw):
    W = make_workload(name, **kw)
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states),
                         threads=8)


def test_empty_and_minimal_inputs(oracle):
    """No edges at all, a sequence without edges beside ordinary ones, and the smallest possible problem."""
    from tests.test_viterbi_gpu import run_cabi_viterbi
    rng = np.random.default_rng(4)
    # E = 0: every frame is empty
    am = rng.uniform(0.1, 3.0, size=(4, 2, 3)).astype(np.float32)
    none = (am, np.zeros((4, 0), np.int32), np.zeros(0, np.float32), np.array([[0, 1], [0, 2]], np.int32),
            np.array([4, 2], np.int32), 3)
    out, loss = check_against_oracle(oracle, none)
    assert (loss == 0).all() and np.isposinf(out).all()
    a, s, code = run_cabi_viterbi(-am, *none[1:])
    assert code == 0 and (a == 0).all() and s.tolist() == [-np.inf, -np.inf]
    # one sequence of the batch has no edges
    W = make_workload("tiny")
    keep = W.edges[3] == 0
    check_against_oracle(oracle, (W.am_scores, W.edges[:, keep].copy(), W.weights[keep].copy(), W.start_end_states,
                                  W.seq_lens, W.n_states))
    # T = B = F = 1, one self-loop on the start = end state
    one = (np.array([[[0.25]]], np.float32), np.array([[0], [0], [0], [0]], np.int32), np.array([0.5], np.float32),
           np.array([[0], [0]], np.int32), np.array([1], np.int32), 1)
    out, loss = check_against_oracle(oracle, one)
    assert loss[0, 0] == pytest.approx(0.75) and out[0, 0, 0] == pytest.approx(0.0, abs=1e-6)


def test_long_sequences(oracle):
    """Twenty thousand frames through a short chain: many renormalisations and progress publications."""
    W = make_workload("monophone", T=20000, B=2, F=120, n_labels=(30, 40))
    W.seq_lens[:] = [20000, 17333]
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=2)


def test_zero_probability_emissions(oracle):
    """am_scores = +inf (probability 0) on some emissions, on whole frames of one emission, and on a
    whole frame: mass flows around them or the sequence has none."""
    W = make_workload("monophone", T=60, B=4, F=40, n_labels=(4, 6))
    am = W.am_scores.copy()
    rng = np.random.default_rng(8)
    mask = rng.random(am.shape) < 0.05
    am[mask] = np.inf
    am[:, 1, 3] = np.inf                      # one emission never possible in sequence 1
    am[10, 2, :] = np.inf                     # nothing possible in frame 10 of sequence 2: no path at all
    out, loss = check_against_oracle(oracle, (am, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states))
    assert (loss[:, 2] == 0).all()


def test_large_batch_of_long_sequences(oracle):
    """More recursion workgroups than compute units and more than 4096 frames: runs on the instance that
    keeps long sequences in double precision."""
    W = make_workload("monophone", T=5000, B=140, F=30, n_labels=(3, 5))
    W.seq_lens[:] = np.random.default_rng(1).integers(4200, 5001, size=140)
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=8)


def test_fast_path_at_capacity(oracle):
    """4096 states and 8190 edges in one sequence: the most the fast kernels hold (one more label and the
    sequence takes the general path)."""
    W = make_workload("cart", T=6200, B=1, F=300, n_labels=(1365, 1365))
    assert W.n_states == 4096 and W.E == 8190
    W.seq_lens[:] = W.T
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=1)


@pytest.mark.parametrize("shuffle", [False, True], ids=["grouped", "shuffled"])
def test_many_short_sequences(oracle, shuffle):
    """More sequences than two large preparation workgroups per compute unit can take in one round: the
    preparation runs with smaller workgroups; edge list grouped by sequence and in random order."""
    W = make_workload("ctc", T=40, B=300, F=400, shuffle_edges=shuffle)
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=8)


@pytest.mark.parametrize("n_labels", [60, 450, 1200], ids=["small", "over-1024-edges", "over-512-classes"])
def test_one_class_on_many_edges(oracle, n_labels):
    """CTC automata put the blank class on every other state: its posterior is a sum over hundreds or
    thousands of edges per frame, which the dense write takes with a whole wave (both of its paths: edges
    in registers, edges staged in passes)."""
    W = make_workload("ctc", T=3 * n_labels, B=2, F=n_labels + 200, n_labels=(n_labels, n_labels + 1))
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=8)


@pytest.mark.parametrize("big_labels,T", [(250, 800), (500, 1550), (1150, 3500)], ids=["1500-edges", "3000-edges", "6900-edges"])
def test_one_large_automaton_among_many_small_ones(oracle, big_labels, T):
    """Twenty small sequences and one large one: few edges per sequence on average, so the preparation runs in
    workgroups of 512 threads, and the large sequence's edges are sorted with four, eight and sixteen keys per thread
    (keys in registers: partners a workgroup apart sit in the same thread)."""
    from tests.test_flat_writer_gpu import merge
    parts = [make_workload("cart", seed=5, T=T, B=20, F=60, n_labels=(3, 9), shuffle_edges=True),
             make_workload("cart", seed=6, T=T, B=1, F=60, n_labels=(big_labels, big_labels))]
    parts[1].seq_lens[:] = T
    am, edges, weights, se, lens, n_states = merge(parts)
    big = int((edges[3] == 20).sum())
    assert edges.shape[1] <= 512 * 21 and big > 1024, (edges.shape, big)
    check_against_oracle(oracle, (am, edges, weights, se, lens, n_states), threads=8)


def test_large_batch_of_tightly_aligned_ctc(oracle):
    """More than 128 sequences (the recursion instance of which two workgroups share a compute unit) of
    CTC automata with 116 labels over up to 850 frames: float state vectors came out at 9e-5 here; the
    small sequences of such batches keep theirs in double."""
    W = make_workload("ctc", seed=2, T=850, B=140, F=300, n_labels=(116, 117))
    out, loss = check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=16)
    want_out, _ = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states, threads=16)
    assert np.abs(posterior(out) - posterior(want_out)).max() < 4e-5
