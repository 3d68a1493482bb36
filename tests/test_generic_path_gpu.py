"""Automata beyond the capacity of the fast kernels (more than 15 edges into or out of a state,
more than 8192 edges, 4096 states or 4096 distinct emissions in one sequence, more emission
classes than the preparation's bitmap holds) take the general path inside the same kernels.  Same parity
bar as everything else, under both schedules, also mixed with ordinary sequences in one batch."""
import numpy as np
import pytest

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import spread_state_ids
from tests.test_fbw_gpu import check_against_oracle, schedule  # noqa: F401  (autouse fixture: both schedules)

pytestmark = pytest.mark.gpu


def fan(rng, T, F, n_mid, seq=0, off=0):
    """start -> n_mid parallel middle states -> end, every middle state with a loop: degree n_mid at
    the start (out) and at the end (in)."""
    frm, to, emis = [], [], []
    s, e = off, off + n_mid + 1
    for i in range(n_mid):
        mid = off + 1 + i
        frm += [s, mid, mid]
        to += [mid, mid, e]
        emis += [int(x) for x in rng.integers(0, F, size=3)]
    n = len(frm)
    edges = np.array([frm, to, emis, [seq] * n], dtype=np.int32)
    return edges, rng.uniform(0.0, 1.5, size=n).astype(np.float32), s, e, n_mid + 2


def test_high_degree_mixed_with_ordinary_sequences(oracle):
    rng = np.random.default_rng(11)
    W = make_workload("tiny")                                  # two ordinary sequences ...
    T, F = W.T, W.F
    e2, w2, s2, t2, n2 = fan(rng, T, F, 20, seq=2, off=W.n_states)          # ... and one with degree 20
    edges = np.concatenate([W.edges, e2], axis=1)
    weights = np.concatenate([W.weights, w2])
    start_end = np.concatenate([W.start_end_states, np.array([[s2], [t2]], np.int32)], axis=1)
    seq_lens = np.concatenate([W.seq_lens, np.array([17], np.int32)])
    am = rng.uniform(0.1, 4.0, size=(T, 3, F)).astype(np.float32)
    am[:, :2] = W.am_scores
    for shuffle in (False, True):
        if shuffle:
            perm = rng.permutation(edges.shape[1])
            edges, weights = edges[:, perm].copy(), weights[perm].copy()
        check_against_oracle(oracle, (am, edges, weights, start_end, seq_lens, W.n_states + n2), bitwise=False)


@pytest.mark.parametrize("kind", ["many_states", "many_edges", "many_emissions"])
def test_large_sequences(oracle, kind):
    """Left-to-right chains beyond one of the per-sequence capacities."""
    if kind == "many_states":       # 4500 states, 9000 edges
        W = make_workload("cart", T=7500, B=1, F=300, n_labels=(1500, 1500))
        W.seq_lens[:] = W.T
    elif kind == "many_edges":      # silence states add edges: > 8192 edges with < 4096 states is not reachable with
        W = make_workload("longform", T=8400, B=2, F=700, n_labels=(1380, 1390))   # chains, so this also has > 4096 states
        W.seq_lens[:] = W.T
    else:                           # 4200 distinct emissions among 1400 labels x 3 states
        W = make_workload("cart", T=8400, B=1, F=50000, n_labels=(1400, 1400))
        W.seq_lens[:] = W.T
    per_seq = W.edges_per_seq()
    print(kind, "edges per sequence", per_seq.tolist(), "states", W.n_states, flush=True)
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), threads=4, bitwise=False)


@pytest.mark.parametrize("F", [24576, 24577, 49153, 100003, 131072, 140000])
def test_many_emission_classes(oracle, F):
    """Long rows (F beyond 24 576) go through the LDS row image of the dense write in tiles of 12 288 floats,
    still on the fast kernels with their fixed summation order; beyond the emission bitmap of the
    preparation (131 072) all sequences take the general path."""
    W = make_workload("cart", T=60, B=3, F=F, n_labels=(10, 15))
    # emission classes at both ends of the rows and on tile boundaries
    for k, em in enumerate([0, 1, F - 1, F - 2, 12287, 12288, 12289, 24575, 24576]):
        if em < F:
            W.edges[2, 3 * k] = em
    check_against_oracle(oracle, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states), bitwise=F <= 131072)


@pytest.mark.parametrize("out_mode", ["neg_log", "neg_prob"])
def test_tiled_rows_in_the_fused_layout(oracle, out_mode):
    """Long rows in (B, T, F) order, every row at another offset within its 128-byte line (F odd)."""
    import torch
    from i6_native_ops_amd.fbw import fbw_loss, core
    W = make_workload("ctc", T=30, B=5, F=45001)
    dev = torch.device("cuda:0")
    fsa = (W.n_states, torch.from_numpy(W.edges).to(dev), torch.from_numpy(W.weights).to(dev),
           torch.from_numpy(W.start_end_states).to(dev))
    seq_lens = torch.from_numpy(W.seq_lens).to(dev)
    want_out, want_loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    if out_mode == "neg_prob":
        log_probs = torch.from_numpy(-W.am_scores).transpose(0, 1).contiguous().to(dev).requires_grad_(True)
        loss = fbw_loss(log_probs, fsa, seq_lens)
        loss.sum().backward()
        np.testing.assert_allclose(loss.detach().cpu().numpy(), want_loss, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(-log_probs.grad.transpose(0, 1).cpu().numpy(), np.exp(-want_out.astype(np.float64)), rtol=0, atol=1e-4)
    else:
        out, loss = core.fbw(torch.from_numpy(W.am_scores).to(dev), fsa[1], fsa[2], fsa[3], seq_lens, W.n_states)
        np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=1e-5, atol=1e-6)
        out = out.cpu().numpy()
        assert (np.isposinf(out) == np.isposinf(want_out)).all()
        np.testing.assert_allclose(np.exp(-out.astype(np.float64)), np.exp(-want_out.astype(np.float64)), rtol=0, atol=1e-4)


def test_status_is_clean_for_general_path():
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    rng = np.random.default_rng(2)
    edges, weights, s, e, n = fan(rng, 12, 9, 30)
    am = rng.uniform(0.1, 3.0, size=(12, 1, 9)).astype(np.float32)
    P = DeviceProblem(am, edges, weights, np.array([[s], [e]], np.int32), np.array([12], np.int32), n)
    P.run(cabi.OUT_PROB)                 # raises on any reported status


@pytest.mark.parametrize("how", ["stride", "permute"])
@pytest.mark.parametrize("name,kw", [("cart", dict(T=80, B=4, F=120)), ("ctc", dict(T=50, B=9, F=60, shuffle_edges=True)),
                                     ("monophone", dict(T=400, B=2, F=70, n_labels=(90, 100)))])
def test_widely_spread_state_ids(oracle, how, name, kw):
    """The reference indexes its state buffers with the ids as they come, so ids need not be compact.
    Sequences whose ids span much more than their number get dense numbers on the device (their rank
    among the ids of the sequence) and stay on the fast kernels; the oracle sees the spread ids as they
    are.  Ids that keep their order give the tables of the compact numbering, hence the same bits."""
    from i6_native_ops_amd import cabi
    from tests.gpu_util import run_cabi
    W = make_workload(name, **kw)
    edges, start_end, n_states = spread_state_ids(W.edges, W.start_end_states, W.n_states, how)
    out, loss = check_against_oracle(oracle, (W.am_scores, edges, W.weights, start_end, W.seq_lens, n_states))
    compact_out, compact_loss = run_cabi(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states,
                                         out_mode=cabi.OUT_NEG_LOG)
    if how == "stride":
        np.testing.assert_array_equal(loss, compact_loss)
        np.testing.assert_array_equal(out, compact_out)
    else:
        np.testing.assert_allclose(loss, compact_loss, rtol=1e-5, atol=1e-6)


def test_widely_spread_state_ids_of_a_large_sequence(oracle):
    """More than 4095 edges: too many ids to sort in LDS; numbers are handed out through a table in the
    workspace and the sequence takes the general path."""
    W = make_workload("cart", T=5200, B=1, F=200, n_labels=(700, 700))
    W.seq_lens[:] = W.T
    assert W.E > 4095
    edges, start_end, n_states = spread_state_ids(W.edges, W.start_end_states, W.n_states, "permute")
    check_against_oracle(oracle, (W.am_scores, edges, W.weights, start_end, W.seq_lens, n_states), bitwise=False)


def test_two_sequences_naming_the_same_states(oracle):
    """Each sequence works on its own copy of the states it names, also when the ids are renumbered: two
    sequences over the same widely spread ids do not disturb each other."""
    W = make_workload("cart", T=40, B=1, F=50)
    edges, start_end, n_states = spread_state_ids(W.edges, W.start_end_states, W.n_states, "stride")
    twice = np.concatenate([edges, edges], axis=1)
    twice[3, edges.shape[1]:] = 1
    am = np.concatenate([W.am_scores, W.am_scores[::-1]], axis=1).copy()
    args1 = (W.am_scores, edges, W.weights, start_end, W.seq_lens, n_states)
    args2 = (am[:, 1:].copy(), edges, W.weights, start_end, W.seq_lens, n_states)
    from tests.gpu_util import run_cabi
    from i6_native_ops_amd import cabi
    post, loss = run_cabi(am, twice, np.concatenate([W.weights, W.weights]), np.concatenate([start_end, start_end], axis=1),
                          np.concatenate([W.seq_lens, W.seq_lens]), n_states, out_mode=cabi.OUT_PROB)
    for b, args in enumerate((args1, args2)):
        want_out, want_loss = oracle.fbw_oracle(*args)
        np.testing.assert_allclose(loss[:, b], want_loss[:, 0], rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(post[:, b], np.exp(-want_out[:, 0].astype(np.float64)), rtol=0, atol=1e-4)


@pytest.mark.parametrize("n_mid", [9, 12, 15, 16])
def test_degree_just_beyond_the_register_tables(oracle, n_mid):
    """Degrees 9 to 15 still run on the table-driven kernels (the table is re-read from memory each frame;
    fixed summation order, so the result is reproducible bit for bit); 16 and more take the general path.
    A hub of that degree inside an ordinary left-to-right automaton, and the bare fan."""
    rng = np.random.default_rng(100 + n_mid)
    W = make_workload("cart", T=90, B=3, F=80, n_labels=(8, 12))
    edges, weights = W.edges.copy(), W.weights.copy()
    for b in range(W.B):                                     # n_mid extra edges into the end state, out of the start state
        states = np.unique(edges[:2, edges[3] == b])
        s, e = int(W.start_end_states[0, b]), int(W.start_end_states[1, b])
        frm = rng.choice(states, size=n_mid); to = rng.choice(states, size=n_mid)
        extra = np.array([np.concatenate([frm, [s] * n_mid]), np.concatenate([[e] * n_mid, to]),
                          rng.integers(0, W.F, size=2 * n_mid), [b] * (2 * n_mid)], dtype=np.int32)
        edges = np.concatenate([edges, extra], axis=1)
        weights = np.concatenate([weights, rng.uniform(0.2, 2.0, size=2 * n_mid).astype(np.float32)])
    check_against_oracle(oracle, (W.am_scores, edges, weights, W.start_end_states, W.seq_lens, W.n_states), bitwise=n_mid <= 15 - 3)
    e2, w2, s2, t2, n2 = fan(rng, 12, 9, n_mid)
    am = rng.uniform(0.1, 3.0, size=(12, 1, 9)).astype(np.float32)
    check_against_oracle(oracle, (am, e2, w2, np.array([[s2], [t2]], np.int32), np.array([12], np.int32), n2), bitwise=n_mid <= 15)
