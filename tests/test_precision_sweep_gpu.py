"""Seeded randomised parity sweep of i6fbw_run against the fp64 oracle, through the C ABI.

The recursion keeps the state vector of a sequence in float or in double depending on its shape
(frames per state, length, batch size: see recurse_workgroup).  This sweep pins the bar -- loss
relative error <= 1e-5, posterior absolute error <= 1e-4 -- on random shapes of all three automaton
families, under both schedules, and on shapes placed on either side of every one of those
decisions: 1024 / 1025 frames, five states for three frames, 256 states with four frames each,
and, for batches of more than 128 sequences (the recursion instance of which two workgroups share a
compute unit, used while the automata are small on average), 383 / 384 frames, more than 1024 frames and more
states than that instance has compute threads; batches of large automata (more than 512 states on
average) run a third instance with fifteen compute waves.  Every case is printed with its errors; the cases beyond the bar fail the test,
and each group of cases also has a tighter bound of its own just above what it measures today, so that a loss of precision
shows long before it reaches the bar.
"""
import numpy as np
import pytest

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import posterior

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
POST_ATOL = 1e-4


def chain_workload(kind, seed, T, B, F, n_labels, lens):
    W = make_workload(kind, seed=seed, T=T, B=B, F=F, n_labels=n_labels)
    lens = np.asarray(lens, dtype=np.int32)
    W.seq_lens[:] = np.resize(lens, B)
    return W


def worst_errors(oracle, W, overlap):
    from i6_native_ops_amd import cabi
    from tests.gpu_util import run_cabi
    args = (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    want_out, want_loss = oracle.fbw_oracle(*args, threads=16)
    cabi.set_overlap(overlap)
    try:
        out, loss = run_cabi(*args, out_mode=cabi.OUT_PROB)
    finally:
        cabi.set_overlap(-1)
    nz = want_loss != 0
    assert (loss[~nz] == 0).all()
    lerr = float(np.max(np.abs(loss[nz] - want_loss[nz]) / np.abs(want_loss[nz]))) if nz.any() else 0.0
    perr = float(np.max(np.abs(out - posterior(want_out))))
    return lerr, perr


def check(oracle, W, overlap, what, failures):
    lerr, perr = worst_errors(oracle, W, overlap)
    print(f"{what}: loss {lerr:.2e} posterior {perr:.2e}", flush=True)
    if not (lerr <= LOSS_RTOL and perr <= POST_ATOL):
        failures.append(f"{what}: loss {lerr:.2e} posterior {perr:.2e}")
    return perr


# (family, labels, frames): states = 3 * labels + 1 for the chains, 2 * labels + 3 for ctc
THRESHOLD_CASES = [
    # 256 / 257 frames (longer sequences always run in double), relaxed alignment
    ("cart", 40, 256), ("cart", 40, 257), ("ctc", 60, 256), ("ctc", 60, 257), ("cart", 59, 400),
    # 1024 / 1025 frames
    ("cart", 100, 1024), ("cart", 100, 1025), ("ctc", 120, 1024), ("ctc", 120, 1025),
    # five states for every three frames: 3 L = 5 S at S = 601, L = 1001.67
    ("cart", 200, 1000), ("cart", 200, 1002), ("cart", 200, 1004), ("monophone", 150, 760),
    # at most 256 states and fewer than four frames per state: S = 250 -> L = 1000
    ("cart", 83, 998), ("cart", 83, 1000), ("cart", 83, 1003), ("cart", 85, 1000), ("ctc", 124, 1000), ("ctc", 126, 1000),
    # 512 / 513 frames (where that limit used to be)
    ("ctc", 120, 512), ("ctc", 120, 513), ("ctc", 200, 512), ("cart", 60, 512), ("cart", 60, 513), ("ctc", 60, 500), ("ctc", 30, 512),
    # tight: one frame per state and a little more
    ("cart", 300, 905), ("cart", 300, 960), ("ctc", 400, 810), ("cart", 340, 1024),
]


@pytest.mark.parametrize("overlap", [0, 1], ids=["single_stream", "overlapped"])
def test_shapes_next_to_the_precision_decisions(oracle, overlap):
    worst, failures = 0.0, []
    for i, (kind, n, L) in enumerate(THRESHOLD_CASES):
        W = chain_workload(kind, 300 + i, T=L + 3, B=3, F=211, n_labels=(n, n), lens=[L, L - 1, L + 2])
        worst = max(worst, check(oracle, W, overlap, f"{kind} labels={n} frames={L}", failures))
    print("worst posterior error", worst)
    assert not failures, failures
    assert worst <= 3e-5        # measured 1.8e-5; 5.8e-5 while the renormalisation still counted states that cannot finish in time


# more than 128 sequences: the instance with 448 compute threads of which two share a compute unit
DENSE_CASES = [
    ("ctc", 48, 255), ("ctc", 48, 256), ("cart", 40, 255), ("cart", 40, 256), ("cart", 59, 380),
    ("ctc", 48, 383), ("ctc", 48, 384), ("ctc", 48, 399), ("ctc", 100, 500), ("cart", 40, 383), ("cart", 40, 384),
    ("ctc", 60, 1024), ("ctc", 60, 1025), ("cart", 120, 1100),
    # more states than the instance has compute threads (several states per thread), short and long
    ("cart", 160, 700), ("cart", 160, 1100), ("ctc", 300, 1100), ("cart", 330, 1030),
]


@pytest.mark.parametrize("overlap", [0, 1], ids=["single_stream", "overlapped"])
def test_large_batches_next_to_the_precision_decisions(oracle, overlap):
    worst, failures = 0.0, []
    for i, (kind, n, L) in enumerate(DENSE_CASES):
        W = chain_workload(kind, 500 + i, T=L + 2, B=130, F=97, n_labels=(n, n), lens=[L, L - 1, L + 1, L - 7])
        worst = max(worst, check(oracle, W, overlap, f"B=130 {kind} labels={n} frames={L}", failures))
    print("worst posterior error", worst)
    assert not failures, failures
    assert worst <= 5e-5        # measured 3.6e-5; 8.2e-5 before (991 states over 1030 frames with 97 emission classes)


def test_large_batch_with_one_sequence_beyond_the_double_capacity_of_its_instance(oracle):
    """129 small sequences and one tight one of 2101 states in a batch of more than 128: the recursion instance
    for such batches has room for 2032 states in double, so the preparation sends it to the general path."""
    from tests.test_flat_writer_gpu import merge
    T = 2150
    small = make_workload("ctc", seed=71, T=T, B=129, F=97, n_labels=(20, 40))
    big = make_workload("cart", seed=72, T=T, B=1, F=97, n_labels=(700, 700))
    big.seq_lens[:] = T - 3
    am, edges, weights, se, lens, n_states = merge([small, big])

    class W:
        pass
    W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states = am, edges, weights, se, lens, n_states
    failures = []
    for overlap in (0, 1):
        check(oracle, W, overlap, f"129 small + 1 of 2101 states, overlap={overlap}", failures)
    assert not failures, failures


def test_large_batch_with_a_few_sequences_of_several_states_per_thread(oracle):
    """A batch of more than 128 sequences runs the recursion instance of which two workgroups share a compute
    unit only while its automata are small on average; this one is (120 small CTC automata), and its ten
    chain automata of 601 states over up to 1100 frames take that instance's path for several states per thread,
    in double."""
    from tests.test_flat_writer_gpu import merge
    T = 1100
    small = make_workload("ctc", seed=81, T=T, B=120, F=97, n_labels=(20, 40))
    mid = make_workload("cart", seed=82, T=T, B=10, F=97, n_labels=(200, 200))
    mid.seq_lens[:] = np.resize(np.asarray([T, T - 1, 700, 1024, 1025], dtype=np.int32), 10)
    am, edges, weights, se, lens, n_states = merge([small, mid])

    class W:
        pass
    W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states = am, edges, weights, se, lens, n_states
    assert n_states <= 448 * 130
    failures = []
    for overlap in (0, 1):
        check(oracle, W, overlap, f"120 small + 10 of 601 states, overlap={overlap}", failures)
    assert not failures, failures


def test_one_large_automaton_of_higher_degree_among_small_ones(oracle):
    """Six small CTC automata and one of 603 states: the batch runs the instance with eight compute waves
    (small automata on average), and the large one, whose final state collects five edges, keeps two states per
    thread with its edges in registers; 1203 states take the table-driven loop."""
    from tests.test_flat_writer_gpu import merge
    failures = []
    for n in (300, 600):
        T = 2 * n + 200
        small = make_workload("ctc", seed=91, T=T, B=6, F=211, n_labels=(30, 50))
        large = make_workload("ctc", seed=92, T=T, B=1, F=211, n_labels=(n, n))
        large.seq_lens[:] = T - 5
        am, edges, weights, se, lens, n_states = merge([small, large])

        class W:
            pass
        W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states = am, edges, weights, se, lens, n_states
        assert n_states <= 512 * 7
        for overlap in (0, 1):
            check(oracle, W, overlap, f"6 small + 1 CTC automaton of {2 * n + 3} states, overlap={overlap}", failures)
    assert not failures, failures


class _Args:
    """the fields of a workload that check() reads"""
    def __init__(self, am, edges, weights, se, lens, n_states):
        self.am_scores, self.edges, self.weights, self.start_end_states, self.seq_lens, self.n_states = am, edges, weights, se, lens, n_states


# bounds of the two groups below: just above what they measure today
PERMUTED_IDS_BOUND = 5e-5          # measured 3.3e-5 (9.9e-5 while the renormalisation went by the ids)
TIGHT_MONOPHONE_BOUND = 3e-5       # measured 1.6e-5 (8.7e-5 in float)


@pytest.mark.parametrize("companions", [0, 90], ids=["large_automata_instance", "two_per_unit_instance"])
@pytest.mark.parametrize("shuffle", [False, True], ids=["edges_in_order", "edges_shuffled"])
def test_tight_chains_under_arbitrary_state_ids(oracle, companions, shuffle):
    """Forty chains of 1021 states over 1021 to 1100 frames whose state ids are drawn at random from a range three times
    as large: nothing about the ids says where a state sits in its automaton.  The renormalisation of the stored
    rows has to find the states that can still matter from the automaton itself (this shape had the worst
    posterior error of all random runs, 9.3e-5, while it looked at the ids).  Alone the batch runs the recursion
    instance for large automata, with ninety small sequences beside it the one of which two workgroups share a
    compute unit."""
    from tests.helpers import spread_state_ids
    from tests.test_flat_writer_gpu import merge
    T = 1100
    parts = [make_workload("cart", seed=955309586, T=T, B=40, F=97, n_labels=(340, 340), shuffle_edges=shuffle)]
    parts[0].seq_lens[:] = np.resize(np.asarray([1100, 1021, 1098, 1050, 1030, 1075, 1023], dtype=np.int32), 40)
    if companions:
        parts.insert(0, make_workload("monophone", seed=371914332, T=T, B=companions, F=97, n_labels=(3, 3), shuffle_edges=True))
        parts[0].seq_lens[:] = T
    am, edges, weights, se, lens, n_states = merge(parts)
    edges, se, n_states = spread_state_ids(edges, se, n_states, "permute", seed=17)
    failures, worst = [], 0.0
    for overlap in (0, 1):
        worst = max(worst, check(oracle, _Args(am, edges, weights, se, lens, n_states), overlap,
                                 f"40 chains of 1021 states, permuted ids, {companions} small beside them, shuffle={shuffle}, overlap={overlap}",
                                 failures))
    assert not failures, failures
    assert worst <= PERMUTED_IDS_BOUND


def test_tight_chain_whose_permuted_ids_span_less_than_twice_its_edges(oracle):
    """One chain of 1021 states over 1100 frames beside eight small sequences, ids permuted over the whole batch: the
    ids of the chain then span about 3500 values -- too few for the sequence to count as one with spread ids (more
    than 2 * edges + 2), too many for the numbering along the automaton, which holds 2048 states, to take the span
    for the number of states (7.9e-5 in the random runs before such a sequence had its ids ranked first)."""
    from tests.helpers import spread_state_ids
    from tests.test_flat_writer_gpu import merge
    T = 1100
    parts = [make_workload("cart", seed=4242, T=T, B=8, F=600, n_labels=(5, 11), shuffle_edges=False),
             make_workload("cart", seed=955309586, T=T, B=1, F=600, n_labels=(340, 340), shuffle_edges=False)]
    for p in parts:
        p.seq_lens[:] = T
    am, edges, weights, se, lens, n_states = merge(parts)
    edges, se, n_states = spread_state_ids(edges, se, n_states, "permute", seed=3)
    big = edges[3] == 8
    span = int(max(edges[0, big].max(), edges[1, big].max()) - min(edges[0, big].min(), edges[1, big].min())) + 1
    assert 2048 < span <= 2 * int(big.sum()) + 2, span             # the case this test is about
    failures, worst = [], 0.0
    for overlap in (0, 1):
        worst = max(worst, check(oracle, _Args(am, edges, weights, se, lens, n_states), overlap,
                                 f"one chain of 1021 states, ids permuted over a batch of nine, overlap={overlap}", failures))
    assert not failures, failures
    assert worst <= PERMUTED_IDS_BOUND


def test_loosely_aligned_sequences_of_400_frames(oracle):
    """Forty chains of up to 177 states and eight of nine states over up to 400 frames: nothing about their shape asks
    for double state vectors, only their length -- the worst case of the random runs while float was kept up to 512
    frames (7.1e-5; 9.8e-6 since it ends at 256)."""
    from tests.test_flat_writer_gpu import merge
    T = 400
    parts = [make_workload("cart", seed=11, T=T, B=8, F=40, n_labels=(2, 3), shuffle_edges=False),
             make_workload("cart", seed=12, T=T, B=40, F=40, n_labels=(30, 59), shuffle_edges=True)]
    am, edges, weights, se, lens, n_states = merge(parts)
    failures, worst = [], 0.0
    for overlap in (0, 1):
        worst = max(worst, check(oracle, _Args(am, edges, weights, se, lens, n_states), overlap,
                                 f"48 loosely aligned chains over up to 400 frames, overlap={overlap}", failures))
    assert not failures, failures
    assert worst <= 3e-5


def test_large_batch_of_tight_monophone_automata(oracle):
    """140 monophone automata of 200 to 400 states over 320 to 400 frames, many of them with barely more frames than
    states, in one batch: the recursion instance of which two workgroups share a compute unit, whose sequences of
    fewer than 384 frames used to keep float state vectors whatever their shape (8.7e-5 in the random runs)."""
    W = make_workload("monophone", seed=14440930, T=400, B=140, F=97, n_labels=(67, 133), shuffle_edges=True)
    # (lengths as drawn, 320 to 400 frames: about a third of the automata have a path at all, most of those a tight one)
    failures, worst = [], 0.0
    for overlap in (0, 1):
        worst = max(worst, check(oracle, W, overlap, f"140 tight monophone automata, overlap={overlap}", failures))
    assert not failures, failures
    assert worst <= TIGHT_MONOPHONE_BOUND


def test_random_shapes(oracle):
    """160 random cases: family, size, tightness of the alignment, edge order, batch size, schedule."""
    rng = np.random.default_rng(20241)
    worst, failures = 0.0, []
    for case in range(160):
        kind = ["cart", "ctc", "monophone"][int(rng.integers(0, 3))]
        n = int(rng.choice([3, 10, 30, 80, 85, 150, 250, 340]))
        states = 3 * n + 1 if kind != "ctc" else 2 * n + 3
        tight = float(rng.choice([1.02, 1.2, 1.6, 1.7, 2.5, 3.9, 4.1, 8.0]))
        L = int(min(2100, max(states + 1, states * tight)))
        B = int(rng.choice([1, 2, 5, 9]))
        F = int(rng.choice([40, 211, 600]))
        lens = [max(states, L - int(x)) for x in rng.integers(0, 6, size=B)]
        W = make_workload(kind, seed=1000 + case, T=L, B=B, F=F, n_labels=(max(1, n - 2), n),
                          shuffle_edges=bool(rng.integers(0, 2)))
        W.seq_lens[:] = np.asarray(lens, dtype=np.int32)
        overlap = int(rng.integers(0, 2))
        worst = max(worst, check(oracle, W, overlap, f"case {case}: {kind} labels<={n} frames={L} B={B} F={F} overlap={overlap}", failures))
    print("worst posterior error", worst)
    assert not failures, failures
    assert worst <= 6e-5        # measured 4.8e-5
