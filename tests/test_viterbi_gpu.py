"""Best-path alignment on the GPU against the oracle: alignment (int32) and scores (fp32 bit
patterns) must be identical, because both sides do the reference's fp32 additions in the
reference's order and max is exact.  Calls go through the C ABI (i6fbw_viterbi) and through the
Python interface that mirrors i6_native_ops.fast_viterbi."""
import numpy as np
import pytest
import torch

from i6_native_ops_amd import cabi
from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import golden
from tests.helpers import spread_state_ids
from tests.helpers import random_fsa
from tests.test_oracle_viterbi import viterbi_fixture

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["single_stream", "overlapped"], autouse=True)
def schedule(request):
    """Every case runs under both schedules of i6fbw_viterbi (search after / beside the gather)."""
    cabi.set_overlap(0 if request.param == "single_stream" else 1)
    yield request.param
    cabi.set_overlap(-1)


def run_cabi_viterbi(am, edges, weights, start_end, seq_lens, n_states, check=True):
    dev = torch.device("cuda:0")
    T, B, F = am.shape
    E = int(edges.shape[1])
    d_am = torch.from_numpy(np.ascontiguousarray(am)).to(dev)
    d_edges = torch.from_numpy(np.ascontiguousarray(edges)).to(dev)
    d_w = torch.from_numpy(np.ascontiguousarray(weights)).to(dev)
    d_se = torch.from_numpy(np.ascontiguousarray(start_end)).to(dev)
    d_len = torch.from_numpy(np.ascontiguousarray(seq_lens)).to(dev)
    align = torch.full((T, B), -7, dtype=torch.int32, device=dev)
    scores = torch.full((B,), 123.0, dtype=torch.float32, device=dev)
    nbytes = cabi.workspace_size(T, B, F, E, n_states)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    print(f"viterbi T={T} B={B} F={F} E={E} S={n_states}", flush=True)
    cabi.viterbi(d_am.data_ptr(), d_am.stride(0), d_am.stride(1), d_edges.data_ptr(), d_edges.stride(0) if E else 0,
                 d_w.data_ptr(), d_se.data_ptr(), d_se.stride(0), d_len.data_ptr(), T, B, F, E, int(n_states),
                 align.data_ptr(), align.stride(0), align.stride(1), scores.data_ptr(), ws.data_ptr(), nbytes, stream)
    code, seq = cabi.read_status(ws.data_ptr(), B, stream)
    if check and code != 0:
        raise cabi.FbwError(code, seq)
    torch.cuda.synchronize()
    return align.cpu().numpy(), scores.cpu().numpy(), code


def assert_identical(got, want):
    (ga, gs), (wa, ws) = got, want
    np.testing.assert_array_equal(ga, wa)
    np.testing.assert_array_equal(gs.view(np.uint32), ws.view(np.uint32))


def test_reference_vector(oracle):
    args = viterbi_fixture()
    align, scores, _ = run_cabi_viterbi(*args)
    assert align[:, 0].tolist() == golden("fast_viterbi")["expected"]["alignment"]            # test/fast_viterbi.py:39
    assert_identical((align, scores), oracle.viterbi_oracle(*args))


@pytest.mark.parametrize("seed", range(20))
def test_random_automata(oracle, seed):
    rng = np.random.default_rng(8100 + seed)
    am, edges, weights, start_end, seq_lens, n_states = random_fsa(rng, B=int(rng.integers(1, 5)), F=int(rng.integers(2, 40)),
                                                                   T=int(rng.integers(1, 12)))
    am = -am
    if seed % 4 == 0:
        seq_lens[0] = 0
    if seed % 5 == 0:
        # coarse values make exact ties between candidates common
        am = np.round(am)
        weights = np.round(weights * 2) / 2
    got = run_cabi_viterbi(am, edges, weights, start_end, seq_lens, n_states)[:2]
    assert_identical(got, oracle.viterbi_oracle(am, edges, weights, start_end, seq_lens, n_states))


def test_hand_worked_cases(oracle):
    """The tie, no-path and zero-length cases that pin the oracle, on the GPU."""
    am = np.zeros((2, 1, 6), dtype=np.float32)
    diamond = np.array([[0, 1, 1, 0], [0, 2, 2, 0], [2, 3, 4, 0], [1, 3, 5, 0]], dtype=np.int32).T.copy()
    a, s, _ = run_cabi_viterbi(am, diamond, np.zeros(4, np.float32), np.array([[0], [3]], np.int32), np.array([2], np.int32), 4)
    assert a[:, 0].tolist() == [2, 4] and s[0] == 0.0
    one = np.array([[0, 1, 5, 0]], dtype=np.int32).T.copy()
    a, s, _ = run_cabi_viterbi(am, one, np.zeros(1, np.float32), np.array([[0], [1]], np.int32), np.array([2], np.int32), 2)
    assert a[:, 0].tolist() == [5, 0] and s[0] == -np.inf
    two = np.array([[0, 0, 1, 0], [1, 2, 2, 1]], dtype=np.int32).T.copy()
    am2 = np.zeros((3, 2, 4), dtype=np.float32)
    a, s, _ = run_cabi_viterbi(am2, two, np.zeros(2, np.float32), np.array([[0, 1], [0, 2]], np.int32), np.array([0, 0], np.int32), 3)
    assert (a == 0).all() and s.tolist() == [0.0, -np.inf]


@pytest.mark.parametrize("name", ["tiny", "monophone", "ctc"])
@pytest.mark.parametrize("shuffle", [False, True])
def test_workloads(oracle, name, shuffle):
    wl = make_workload(name, shuffle_edges=shuffle)
    am, w = -wl.am_scores, -wl.weights
    got = run_cabi_viterbi(am, wl.edges, w, wl.start_end_states, wl.seq_lens, wl.n_states)[:2]
    want = oracle.viterbi_oracle(am, wl.edges, w, wl.start_end_states, wl.seq_lens, wl.n_states)
    assert np.isfinite(want[1]).all()
    assert_identical(got, want)


@pytest.mark.parametrize("kind", ["cart_small", "large_states", "large_emissions", "huge_states", "ctc_two_per_thread", "ctc_table"])
def test_size_classes(oracle, kind):
    """Chains that take the one-state-per-thread path, the four-states-per-thread path (more than 512
    states or distinct emissions) and the table-in-memory path (more than 2048 states); CTC automata
    (five edges into the final state) of 603 states -- two per thread, edges in registers -- and of 1203."""
    if kind.startswith("ctc"):
        n = 300 if kind == "ctc_two_per_thread" else 600
        wl = make_workload("ctc", T=2 * n + 150, B=2, F=700, n_labels=(n, n))
    elif kind == "cart_small":
        wl = make_workload("cart", T=300, B=4, F=12001, n_labels=(60, 90))
    elif kind == "large_states":
        wl = make_workload("cart", T=900, B=2, F=300, n_labels=(250, 280))
    elif kind == "large_emissions":
        wl = make_workload("cart", T=900, B=2, F=12001, n_labels=(250, 280))
    else:
        wl = make_workload("cart", T=2200, B=1, F=300, n_labels=(700, 710))
    wl.seq_lens[:] = wl.T          # long enough for the longest chain
    am, w = -wl.am_scores, -wl.weights
    got = run_cabi_viterbi(am, wl.edges, w, wl.start_end_states, wl.seq_lens, wl.n_states)[:2]
    assert_identical(got, oracle.viterbi_oracle(am, wl.edges, w, wl.start_end_states, wl.seq_lens, wl.n_states))


def test_one_large_automaton_among_many_small_ones(oracle):
    """Few edges per sequence on average (preparation in workgroups of 512 threads) and one sequence of 3000: its
    edges are sorted with eight keys per thread; the alignment stays bit-identical."""
    from tests.test_flat_writer_gpu import merge
    T = 1550
    parts = [make_workload("cart", seed=5, T=T, B=20, F=60, n_labels=(3, 9), shuffle_edges=True),
             make_workload("cart", seed=6, T=T, B=1, F=60, n_labels=(500, 500))]
    parts[1].seq_lens[:] = T
    am, edges, weights, se, lens, n_states = merge(parts)
    got = run_cabi_viterbi(-am, edges, -weights, se, lens, n_states)[:2]
    assert_identical(got, oracle.viterbi_oracle(-am, edges, -weights, se, lens, n_states))


def test_device_status():
    """An index out of range is reported; the sequence gets score NaN and an all-zero alignment."""
    edges = np.array([[0, 1, 1, 0], [1, 1, 9, 0]], dtype=np.int32).T.copy()      # emission class 9 of 4
    am = np.zeros((2, 1, 4), dtype=np.float32)
    a, s, code = run_cabi_viterbi(am, edges, np.zeros(2, np.float32), np.array([[0], [1]], np.int32),
                                  np.array([2], np.int32), 2, check=False)
    assert code == -14 and np.isnan(s[0]) and (a == 0).all()


@pytest.mark.parametrize("how", ["stride", "permute"])
def test_widely_spread_state_ids(oracle, how):
    """State ids of a sequence far apart get dense numbers on the device; the result is that of the same
    automata with compact ids, bit for bit."""
    wl = make_workload("cart", T=60, B=5, F=90)
    am, w = -wl.am_scores, -wl.weights
    want = oracle.viterbi_oracle(am, wl.edges, w, wl.start_end_states, wl.seq_lens, wl.n_states)
    edges, start_end, n_states = spread_state_ids(wl.edges, wl.start_end_states, wl.n_states, how)
    assert_identical(run_cabi_viterbi(am, edges, w, start_end, wl.seq_lens, n_states)[:2], want)
    assert_identical(oracle.viterbi_oracle(am, edges, w, start_end, wl.seq_lens, n_states), want)


@pytest.mark.parametrize("kind", ["degree", "degree12", "ties12", "many_states", "many_classes", "ties"])
def test_general_path(oracle, kind):
    """Beyond the capacity of the fast kernels (more than 15 edges into a state (9 to 15: tables re-read per frame), more than 4096 states,
    more emission classes than the bitmap holds): same bits as the oracle, ties included."""
    rng = np.random.default_rng(77)
    if kind in ("degree", "ties", "degree12", "ties12"):        # degree 12: tables re-read per frame; 25: general path
        T, F, n_mid = 14, 9, (12 if kind.endswith("12") else 25)
        frm, to, emis = [], [], []
        for i in range(n_mid):
            frm += [0, 1 + i, 1 + i]
            to += [1 + i, 1 + i, n_mid + 1]
            emis += [int(x) for x in rng.integers(0, F, size=3)]
        edges = np.array([frm, to, emis, [0] * len(frm)], dtype=np.int32)
        weights = rng.uniform(-1.5, 0.0, size=len(frm)).astype(np.float32)
        am = -rng.uniform(0.1, 3.0, size=(T, 1, F)).astype(np.float32)
        if kind.startswith("ties"):
            weights[:] = -0.5
            am = np.round(am)
        args = (am, edges, weights, np.array([[0], [n_mid + 1]], np.int32), np.array([11], np.int32), n_mid + 2)
    elif kind == "many_states":
        W = make_workload("cart", T=5000, B=1, F=300, n_labels=(1500, 1500))
        W.seq_lens[:] = W.T
        args = (-W.am_scores, W.edges, -W.weights, W.start_end_states, W.seq_lens, W.n_states)
    else:
        W = make_workload("cart", T=60, B=3, F=140000, n_labels=(10, 15))
        args = (-W.am_scores, W.edges, -W.weights, W.start_end_states, W.seq_lens, W.n_states)
    got = run_cabi_viterbi(*args)[:2]
    want = oracle.viterbi_oracle(*args)
    assert np.isfinite(want[1]).all()
    assert_identical(got, want)


def test_python_interface(oracle):
    """align_viterbi(log_probs (B,T,F), fsa, seq_lens) -> ((B,T) int32, (B,)) as in
    i6_native_ops/fast_viterbi/__init__.py:23-47, and core.fast_viterbi on (T,B,F)."""
    from i6_native_ops_amd.fast_viterbi import align_viterbi, core
    am, edges, weights, start_end, seq_lens, n = viterbi_fixture()
    dev = "cuda:0"
    log_probs = torch.from_numpy(am).to(dev).transpose(0, 1).contiguous()       # (B, T, F)
    fsa = (n, torch.from_numpy(edges).to(dev), torch.from_numpy(weights).to(dev), torch.from_numpy(start_end).to(dev))
    output, scores = align_viterbi(log_probs, fsa, torch.from_numpy(seq_lens).to(dev))
    assert output.shape == (1, 5) and output.dtype == torch.int32 and scores.shape == (1,)
    assert output[0].cpu().tolist() == golden("fast_viterbi")["expected"]["alignment"]
    want = oracle.viterbi_oracle(am, edges, weights, start_end, seq_lens, n)
    assert float(scores[0]) == float(want[1][0])

    wl = make_workload("monophone")
    lp = torch.from_numpy(-wl.am_scores).to(dev).transpose(0, 1).contiguous()
    fsa = (wl.n_states, torch.from_numpy(wl.edges).to(dev), torch.from_numpy(-wl.weights).to(dev),
           torch.from_numpy(wl.start_end_states).to(dev))
    lens = torch.from_numpy(wl.seq_lens).to(dev)
    out_bt, sc = align_viterbi(lp, fsa, lens)
    out_tb, sc2 = core.fast_viterbi(lp.transpose(0, 1).contiguous(), fsa[1], fsa[2], fsa[3], lens, wl.n_states)
    want = oracle.viterbi_oracle(-wl.am_scores, wl.edges, -wl.weights, wl.start_end_states, wl.seq_lens, wl.n_states)
    np.testing.assert_array_equal(out_bt.cpu().numpy(), want[0].T)
    np.testing.assert_array_equal(out_tb.cpu().numpy(), want[0])
    np.testing.assert_array_equal(sc.cpu().numpy(), want[1])
    np.testing.assert_array_equal(sc2.cpu().numpy(), want[1])
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        core.fast_viterbi(lp.cpu(), fsa[1], fsa[2], fsa[3], lens, wl.n_states)
