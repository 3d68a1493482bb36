"""Pins the CPU oracle (oracle/fbw_oracle.c) without running the reference:
closed forms on the reference's fixture, brute force, library special cases,
finite differences and invariants.  Each check is chosen so that a dropped
term, a wrong sign or index, or swapped from/to fails it."""
import numpy as np
import pytest
import torch

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import brute_force, posterior, random_fsa, reference_fixture


@pytest.mark.parametrize("prec,tol", [("f64", 1e-9), ("f32", 2e-6)])
def test_reference_fixture_closed_form(oracle, prec, tol):
    # 5 accepting paths with sum of path probabilities 0.73224;
    # the three unit weights add 1 per frame: NLL = 5 - ln 0.73224.
    out, loss = oracle.fbw_oracle(*reference_fixture(5), precision=prec)
    p = [[.9, .1], [.9, .1], [.4, .6], [.1, .9], [.1, .9]]
    # a path emits label 0 on its first k frames (k = 1..5, the frames spent leaving state 0,
    # the last of them on the 0->1 edge) and label 1 on the rest
    paths = [float(np.prod([p[t][0 if t < k else 1] for t in range(5)])) for k in range(1, 6)]
    total = sum(paths)
    assert abs(total - 0.73224) < 1e-5
    np.testing.assert_allclose(loss[:, 0], 5 - np.log(total), rtol=0, atol=max(tol, 2e-7) * 5)
    want = np.array([[1, 0], [.9402655, .0597345], [.4026549, .5973451], [.0442478, .9557522], [.0044248, .9955752]])
    np.testing.assert_allclose(posterior(out)[:, 0], want, atol=2e-7 + tol)
    # row-sum invariant of test/fbw.py:60-64
    np.testing.assert_allclose(posterior(out).sum(-1), 1.0, atol=1e-6)


def test_reference_fixture_shorter_seq_len(oracle):
    out, loss = oracle.fbw_oracle(*reference_fixture(4))
    np.testing.assert_allclose(loss[:, 0], [4 - np.log(0.81)] * 4 + [0.0], atol=1e-7)
    want = np.array([[1, 0], [.94, .06], [.4, .6], [.04, .96], [0, 0]])
    np.testing.assert_allclose(posterior(out)[:, 0], want, atol=2e-7)
    assert np.isinf(out[4]).all() and (out[4] > 0).all()


@pytest.mark.parametrize("seq_len", [0, 6, -1])
def test_degenerate_seq_len_gives_zero_loss_and_inf_out(oracle, seq_len):
    # beta is never seeded when seq_len is 0 or > T (fbw_op.cu:61-69,339-341)
    out, loss = oracle.fbw_oracle(*reference_fixture(seq_len))
    assert (loss == 0).all()
    assert np.isposinf(out).all()


@pytest.mark.parametrize("seed", range(40))
def test_brute_force_random_automata(oracle, seed):
    rng = np.random.default_rng(seed)
    args = random_fsa(rng, B=int(rng.integers(1, 4)), F=int(rng.integers(1, 5)), T=int(rng.integers(1, 7)))
    out, loss = oracle.fbw_oracle(*args)
    want_loss, want_post = brute_force(*args)
    np.testing.assert_allclose(loss, want_loss, atol=1e-9)
    np.testing.assert_allclose(posterior(out), want_post, atol=1e-6)
    # +inf exactly where nothing contributes
    assert (np.isposinf(out) == (want_post == 0)).all() or np.allclose(posterior(out), want_post, atol=1e-12)
    out32, loss32 = oracle.fbw_oracle(*args, precision="f32")
    np.testing.assert_allclose(loss32, want_loss, atol=2e-5)
    np.testing.assert_allclose(posterior(out32), want_post, atol=2e-5)


def test_threaded_partition_equals_global_sweep(oracle):
    W = make_workload("monophone", T=60, B=5, F=30, shuffle_edges=True)
    a = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states, threads=1)
    b = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states, threads=4)
    np.testing.assert_array_equal(a[0], b[0])
    np.testing.assert_array_equal(a[1], b[1])


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_ctc_topology_equals_torch_ctc_loss(oracle, seed):
    W = make_workload("ctc", seed=seed, T=24, B=4, F=7, n_labels=(2, 6))
    # rebuild the label sequences from the automaton: states v, (blank,label)*, blank, x
    out, loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    log_probs = torch.tensor(-W.am_scores, dtype=torch.float64, requires_grad=True)  # [T,B,F]
    targets, tlens = [], []
    for b in range(W.B):
        v, x = W.start_end_states[:, b]
        labels = []
        for s in range(v + 1, x):
            # emission of state s = emission of its loop edge
            e = np.where((W.edges[0] == s) & (W.edges[1] == s))[0][0]
            if (s - v - 1) % 2 == 1:
                labels.append(int(W.edges[2, e]))
        targets += labels
        tlens.append(len(labels))
    nll = torch.nn.functional.ctc_loss(log_probs, torch.tensor(targets), torch.tensor(W.seq_lens, dtype=torch.long),
                                       torch.tensor(tlens), blank=0, reduction="none", zero_infinity=False)
    for b in range(W.B):
        L = W.seq_lens[b]
        np.testing.assert_allclose(loss[:L, b], nll[b].item(), rtol=1e-10)
        assert (loss[L:, b] == 0).all()
    nll.sum().backward()
    # torch's CTC backward folds the log-softmax in: grad = softmax - posterior on valid
    # frames (our log_probs are normalised), 0 on padded frames
    want = np.exp(-W.am_scores.astype(np.float64)) - log_probs.grad.numpy()
    for b in range(W.B):
        want[W.seq_lens[b]:, b] = 0
    np.testing.assert_allclose(posterior(out), want, atol=1e-6)


def test_linear_hmm_equals_dense_log_matrix_chain(oracle):
    from scipy.special import logsumexp
    W = make_workload("tiny", seed=7)
    out, loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    for b in range(W.B):
        L = int(W.seq_lens[b])
        sel = W.edges[3] == b
        S = W.n_states
        logalpha = np.full(S, -np.inf)
        logalpha[W.start_end_states[0, b]] = 0.0
        for t in range(L):
            M = np.full((S, S), -np.inf)           # log transition matrix of frame t
            for f, to, em, w in zip(W.edges[0, sel], W.edges[1, sel], W.edges[2, sel], W.weights[sel]):
                M[f, to] = np.logaddexp(M[f, to], -(float(w) + float(W.am_scores[t, b, em])))
            logalpha = logsumexp(logalpha[:, None] + M, axis=0)
        np.testing.assert_allclose(loss[:L, b], -logalpha[W.start_end_states[1, b]], rtol=1e-12)


def test_gradient_of_loss_is_posterior_by_finite_differences(oracle):
    rng = np.random.default_rng(3)
    W = make_workload("monophone", seed=11, T=12, B=2, F=9, n_labels=(1, 2))
    base = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    post = posterior(base[0])
    am64 = W.am_scores.astype(np.float64)
    eps = 2.0 ** -7        # exactly representable step; am stays float32-exact
    for _ in range(25):
        t, b, f = int(rng.integers(0, W.T)), int(rng.integers(0, W.B)), int(rng.integers(0, W.F))
        up, dn = W.am_scores.copy(), W.am_scores.copy()
        up[t, b, f] += eps
        dn[t, b, f] -= eps
        lu = oracle.fbw_oracle(up, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)[1][0, b]
        ld = oracle.fbw_oracle(dn, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)[1][0, b]
        h = float(up[t, b, f]) - float(dn[t, b, f])
        # d NLL / d am[t,b,f] = posterior[t,b,f]
        assert abs((lu - ld) / h - post[t, b, f]) < 5e-4, (t, b, f)


@pytest.mark.parametrize("name,kw", [("tiny", {}), ("monophone", dict(T=80, B=6, F=60)),
                                     ("cart", dict(T=100, B=4, F=500)), ("ctc", dict(T=40, B=8, F=50)),
                                     ("longform", dict(T=200, B=2, F=300))])
def test_invariants_on_workloads(oracle, name, kw):
    W = make_workload(name, **kw)
    args = (W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    out, loss = oracle.fbw_oracle(W.am_scores, *args)
    post = posterior(out)
    for b in range(W.B):
        L = int(W.seq_lens[b])
        assert L <= W.T
        np.testing.assert_allclose(post[:L, b].sum(-1), 1.0, atol=1e-5)      # test/fbw.py:60-64
        assert (post[L:, b] == 0).all() and (loss[L:, b] == 0).all()
        assert np.ptp(loss[:L, b]) < 1e-7 * abs(loss[0, b])                    # same NLL in every valid frame
        used = np.zeros(W.F, bool)
        used[W.edges[2, W.edges[3] == b]] = True
        assert np.isposinf(out[:, b][:, ~used]).all()
    # invariance to edge order
    perm = np.random.default_rng(0).permutation(W.E)
    out2, loss2 = oracle.fbw_oracle(W.am_scores, np.ascontiguousarray(W.edges[:, perm]), W.weights[perm].copy(),
                                    *args[2:])
    np.testing.assert_allclose(loss2, loss, rtol=1e-12)
    np.testing.assert_allclose(posterior(out2), post, atol=5e-7)  # out is stored as float32
    # adding c to every weight adds c*seq_len to the loss and leaves posteriors alone
    c = 0.375
    out3, loss3 = oracle.fbw_oracle(W.am_scores, W.edges, W.weights + np.float32(c), *args[2:])
    for b in range(W.B):
        L = int(W.seq_lens[b])
        np.testing.assert_allclose(loss3[:L, b], loss[:L, b] + c * L, rtol=1e-6)
    np.testing.assert_allclose(posterior(out3), post, atol=1e-5)
    # f32 port agrees with the f64 oracle on these small cases
    out4, loss4 = oracle.fbw_oracle(W.am_scores, *args, precision="f32")
    np.testing.assert_allclose(loss4, loss, rtol=2e-5, atol=1e-4)
    np.testing.assert_allclose(posterior(out4), post, atol=3e-3)
