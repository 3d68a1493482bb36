"""Device-side automaton builders (i6fbw_build_ctc_fsa / i6fbw_build_hmm_fsa) and padding edges.

The reference has no builders; they are pinned by (1) torch.nn.functional.ctc_loss on the CPU:
the full-sum loss over the built CTC automaton must equal it, (2) element-wise equality with the
host-side generators of the benchmark workloads, which the oracle tests pin in the same way."""
import numpy as np
import pytest
import torch

from i6_native_ops_amd.fbw.workloads import _assemble, _ctc, _hmm_chain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ragged(rng, B, Lmax, lo, hi, min_len=0):
    lens = rng.integers(min_len, Lmax + 1, size=B).astype(np.int32)
    lab = rng.integers(lo, hi, size=(B, Lmax)).astype(np.int32)
    return lab, lens


def trimmed(fsa, totals):
    n_edges, n_states = (int(x) for x in totals.cpu())
    _, edges, weights, start_end = fsa
    return n_states, edges[:, :n_edges].cpu().numpy(), weights[:n_edges].cpu().numpy(), start_end.cpu().numpy()


@pytest.mark.parametrize("seed", range(4))
def test_ctc_builder_matches_host_generator(seed):
    from i6_native_ops_amd.fsa import ctc_fsa
    rng = np.random.default_rng(300 + seed)
    B, Lmax = int(rng.integers(1, 40)), int(rng.integers(1, 12))
    lab, lens = ragged(rng, B, Lmax, 1, 4)          # few symbols: many repeated neighbours (no skip edge there)
    if seed == 0:
        lens[0] = 0
    fsa, totals = ctc_fsa(torch.from_numpy(lab).to(DEV), torch.from_numpy(lens).to(DEV), blank=0, return_totals=True)
    n_states, edges, weights, start_end = trimmed(fsa, totals)
    autos = [_ctc(lab[b, :lens[b]].tolist(), blank=0) for b in range(B)]
    want = _assemble("x", autos, np.ones(B), 1, B, 4, rng, 1.0, False, False)
    assert n_states == want.n_states
    np.testing.assert_array_equal(edges, want.edges)
    np.testing.assert_array_equal(weights, want.weights)
    np.testing.assert_array_equal(start_end, want.start_end_states)
    # the rest of the capacity is padding
    assert (fsa[1][3, edges.shape[1]:] == -1).all() and fsa[0] >= n_states


def test_ctc_loss_equals_torch(oracle):
    """fbw_loss over the built automaton (used at full capacity, padding edges included) against
    torch's CTC loss and its gradient on the CPU."""
    from i6_native_ops_amd.fbw import fbw_loss
    from i6_native_ops_amd.fsa import ctc_fsa
    rng = np.random.default_rng(17)
    B, T, F, Lmax = 6, 40, 9, 7
    lab, lens = ragged(rng, B, Lmax, 1, F, min_len=1)
    seq_lens = rng.integers(2 * Lmax + 1, T + 1, size=B).astype(np.int32)
    logits = rng.standard_normal((B, T, F)).astype(np.float32)
    log_probs = torch.from_numpy(logits).log_softmax(-1)

    lp = log_probs.to(DEV).requires_grad_(True)
    fsa = ctc_fsa(torch.from_numpy(lab).to(DEV), torch.from_numpy(lens).to(DEV), blank=0)
    loss = fbw_loss(lp, fsa, torch.from_numpy(seq_lens).to(DEV))          # (T, B)
    loss.sum().backward()

    ref_lp = log_probs.clone().requires_grad_(True)
    ref = torch.nn.functional.ctc_loss(ref_lp.transpose(0, 1), torch.from_numpy(lab).long(), torch.from_numpy(seq_lens).long(),
                                       torch.from_numpy(lens).long(), blank=0, reduction="none", zero_infinity=False)
    ref.sum().backward()
    np.testing.assert_allclose(loss[0].detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-5)
    # torch's ctc_loss backward returns softmax - posterior (it folds the log-softmax in); ours is -posterior
    got = lp.grad.cpu().numpy()
    want = ref_lp.grad.numpy() - np.exp(log_probs.numpy())
    for b in range(B):
        np.testing.assert_allclose(got[b, :seq_lens[b]], want[b, :seq_lens[b]], atol=1e-4)
        assert (got[b, seq_lens[b]:] == 0).all()


@pytest.mark.parametrize("table", [False, True])
def test_hmm_builder_matches_host_generator(table):
    from i6_native_ops_amd.fsa import hmm_fsa
    rng = np.random.default_rng(41)
    B, Lmax, spl, n_labels = 9, 13, 3, 20
    lab, lens = ragged(rng, B, Lmax, 0, n_labels, min_len=1)
    tab = rng.integers(0, 500, size=n_labels * spl).astype(np.int32) if table else None
    fsa, totals = hmm_fsa(torch.from_numpy(lab).to(DEV), torch.from_numpy(lens).to(DEV), states_per_label=spl,
                          loop_weight=0.25, forward_weight=1.5,
                          emission_table=torch.from_numpy(tab).to(DEV) if table else None, return_totals=True)
    n_states, edges, weights, start_end = trimmed(fsa, totals)
    autos = []
    for b in range(B):
        idx = [int(l) * spl + k for l in lab[b, :lens[b]] for k in range(spl)]
        emis = [int(tab[i]) for i in idx] if table else idx
        autos.append(_hmm_chain(emis, lambda: 0.25, lambda: 1.5))
    want = _assemble("x", autos, np.ones(B), 1, B, 600, rng, 1.0, False, False)
    assert n_states == want.n_states
    np.testing.assert_array_equal(edges, want.edges)
    np.testing.assert_array_equal(weights, want.weights)
    np.testing.assert_array_equal(start_end, want.start_end_states)
    assert (fsa[1][3, edges.shape[1]:] == -1).all()


def test_padding_edges_are_ignored(oracle):
    """An edge list with padding edges (sequence index -1) at its end, and shuffled among the others,
    gives the results of the list without them -- full sum and best path."""
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw.workloads import make_workload
    from tests.gpu_util import run_cabi
    from tests.test_viterbi_gpu import run_cabi_viterbi
    W = make_workload("tiny")
    want_out, want_loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    pad = np.zeros((4, 37), dtype=np.int32)
    pad[3] = -1
    rng = np.random.default_rng(3)
    for shuffle in (False, True):
        edges = np.concatenate([W.edges, pad], axis=1)
        weights = np.concatenate([W.weights, np.zeros(37, np.float32)])
        if shuffle:
            perm = rng.permutation(edges.shape[1])
            edges, weights = edges[:, perm].copy(), weights[perm].copy()
        out, loss = run_cabi(W.am_scores, edges, weights, W.start_end_states, W.seq_lens, W.n_states + 11, cabi.OUT_PROB)
        np.testing.assert_allclose(loss, want_loss, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(out, np.exp(-want_out.astype(np.float64)), atol=1e-4)
        if not shuffle:        # the best path breaks ties by edge position, which a shuffle changes
            got = run_cabi_viterbi(-W.am_scores, edges, -weights, W.start_end_states, W.seq_lens, W.n_states + 11)[:2]
            want = oracle.viterbi_oracle(-W.am_scores, W.edges, -W.weights, W.start_end_states, W.seq_lens, W.n_states)
            np.testing.assert_array_equal(got[0], want[0])
            np.testing.assert_array_equal(got[1], want[1])
