"""The configurations of the benchmark at their full sizes: size-independent properties of the
result (every valid row of the posterior sums to 1, the loss is the same in every valid frame of a
sequence and 0 after it, holes exactly where no edge of the sequence carries the emission, padding
rows empty, result independent of the edge order) and, since the CPU oracle finishes them in
seconds with a few threads, the full comparison too."""
import numpy as np
import pytest
import torch

from i6_native_ops_amd import cabi
from i6_native_ops_amd.fbw.workloads import make_workload
from tests.gpu_util import DeviceProblem

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["cart", "monophone", "ctc", "longform"])
def test_full_size(oracle, name):
    W = make_workload(name)
    print(f"full size {name}: T={W.T} B={W.B} F={W.F} E={W.E}", flush=True)
    P = DeviceProblem(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    post, loss = P.run(cabi.OUT_PROB)
    torch.cuda.synchronize()
    lens = torch.from_numpy(W.seq_lens).to(post.device)
    valid = torch.arange(W.T, device=post.device)[:, None] < lens[None, :]            # (T, B)

    rowsum = post.sum(-1, dtype=torch.float64)
    assert torch.all((rowsum[valid] - 1.0).abs() < 1e-4)                              # test/fbw.py:60-64
    assert torch.all(rowsum[~valid] == 0)
    assert torch.all(post >= 0) and torch.all(post <= 1.0 + 1e-5)
    # loss: one value per sequence, repeated in its valid frames, 0 afterwards
    first = loss[0][None, :].expand_as(loss)
    assert torch.all(((loss - first).abs() <= 1e-5 * first.abs())[valid])
    assert torch.all(loss[~valid] == 0)
    # holes: posterior mass only on emissions that some edge of the sequence carries
    allowed = torch.zeros((W.B, W.F), dtype=torch.bool, device=post.device)
    allowed[torch.from_numpy(W.edges[3].astype(np.int64)).to(post.device),
            torch.from_numpy(W.edges[2].astype(np.int64)).to(post.device)] = True
    assert torch.all(post.amax(0)[~allowed] == 0)

    # the oracle on the whole problem
    want_out, want_loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens,
                                            W.n_states, threads=min(16, W.B))
    np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=1e-5, atol=1e-6)
    got = post.cpu().numpy()
    worst = 0.0
    for t0 in range(0, W.T, 100):                       # in slices: exp() of the whole tensor at once is 12 GB in float64
        ref = np.exp(-want_out[t0:t0 + 100].astype(np.float64))
        worst = max(worst, float(np.abs(got[t0:t0 + 100] - ref).max()))
    print(f"full size {name}: worst posterior error {worst:.1e}", flush=True)
    assert worst <= 1e-4
    del got, want_out

    # same problem with the edge list shuffled: bitwise the same loss rows up to summation order,
    # checked to the parity tolerance
    rng = np.random.default_rng(5)
    perm = rng.permutation(W.E)
    P2 = DeviceProblem(W.am_scores, W.edges[:, perm].copy(), W.weights[perm].copy(), W.start_end_states, W.seq_lens,
                       W.n_states)
    post2, loss2 = P2.run(cabi.OUT_PROB)
    assert torch.all((loss2 - loss).abs() <= 1e-5 * loss.abs() + 1e-6)
    assert float((post2 - post).abs().max()) <= 1e-4


@pytest.mark.parametrize("name", ["cart", "ctc"])
def test_full_size_neg_log(oracle, name):
    """The -log output (what fbw_core.fbw returns, fbw_op.cu:366-377,392) at full size: the values themselves in the log
    domain, and +inf in exactly the oracle's places -- the reference adds in log space (fbw_op.cu:39-59,137-153) and has
    a finite -log wherever some edge is alive, far below the range of a float posterior."""
    W = make_workload(name)
    print(f"full size -log {name}: T={W.T} B={W.B} F={W.F} E={W.E}", flush=True)
    P = DeviceProblem(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    out, loss = P.run(cabi.OUT_NEG_LOG)
    torch.cuda.synchronize()
    out, loss = out.clone(), loss.clone()          # (the problem's buffers are written again below)
    want_out, want_loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens,
                                            W.n_states, threads=min(16, W.B))
    np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=1e-5, atol=1e-6)
    got = out.cpu().numpy()
    atol = 2e-3 + 1.2e-7 * float(np.abs(want_loss).max())      # a large -log is the difference of two numbers of the size of the loss
    n_fin = n_deep = 0
    for t0 in range(0, W.T, 100):
        g, w = got[t0:t0 + 100], want_out[t0:t0 + 100]
        fin = np.isfinite(w)
        assert (np.isposinf(g) == ~fin).all(), t0
        np.testing.assert_allclose(g[fin], w[fin], rtol=2e-5, atol=atol)
        n_fin += int(fin.sum())
        n_deep += int((w[fin] > 88.0).sum())
    print(f"full size -log {name}: {n_fin} finite elements, {n_deep} of them beyond the range of a float posterior", flush=True)
    assert n_deep > 0       # the case the log-space sums are there for
    # the posterior mode on the same inputs: same loss to rounding, exp(-out) = posterior
    post, loss1 = P.run(cabi.OUT_PROB)
    torch.cuda.synchronize()
    assert torch.all((loss1 - loss).abs() <= 1e-6 * loss.abs())
    assert float((torch.exp(-out) - post).abs().max()) <= 2e-6


def test_full_size_best_path(oracle):
    """Best path on the headline automata: bit-identical to the oracle, and the path's own score,
    re-accumulated in float64 along the alignment, matches the reported score."""
    W = make_workload("cart")
    dev = torch.device("cuda:0")
    am = torch.from_numpy(-W.am_scores).to(dev)
    d = dict(edges=torch.from_numpy(W.edges).to(dev), w=torch.from_numpy(-W.weights).to(dev),
             se=torch.from_numpy(W.start_end_states).to(dev), lens=torch.from_numpy(W.seq_lens).to(dev))
    align = torch.empty((W.T, W.B), dtype=torch.int32, device=dev)
    scores = torch.empty((W.B,), dtype=torch.float32, device=dev)
    nbytes = cabi.workspace_size(W.T, W.B, W.F, W.E, W.n_states)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    cabi.viterbi(am.data_ptr(), am.stride(0), am.stride(1), d["edges"].data_ptr(), d["edges"].stride(0), d["w"].data_ptr(),
                 d["se"].data_ptr(), d["se"].stride(0), d["lens"].data_ptr(), W.T, W.B, W.F, W.E, W.n_states,
                 align.data_ptr(), align.stride(0), align.stride(1), scores.data_ptr(), ws.data_ptr(), nbytes, stream)
    assert cabi.read_status(ws.data_ptr(), W.B, stream) == (0, -1)
    want_align, want_scores = oracle.viterbi_oracle(-W.am_scores, W.edges, -W.weights, W.start_end_states, W.seq_lens,
                                                    W.n_states)
    np.testing.assert_array_equal(align.cpu().numpy(), want_align)
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    # emission scores along the alignment are an upper part of the path score: score - sum(am) = sum of edge weights <= 0
    a = align.cpu().numpy()
    for b in range(0, W.B, 8):
        L = int(W.seq_lens[b])
        em = float((-W.am_scores[np.arange(L), b, a[:L, b]]).astype(np.float64).sum())
        assert float(scores[b]) <= em + 1e-3


def _check_sequences_against_oracle(oracle, W, am, post, loss, which):
    """The oracle on a few sequences of a batch whose scores live on the device only."""
    which = np.asarray(which)
    am_sub = np.ascontiguousarray(am[:, torch.from_numpy(which).to(am.device), :].cpu().numpy())
    keep = np.isin(W.edges[3], which)
    edges = W.edges[:, keep].copy()
    edges[3] = np.searchsorted(which, edges[3])
    want_out, want_loss = oracle.fbw_oracle(am_sub, edges, W.weights[keep].copy(), W.start_end_states[:, which].copy(),
                                            W.seq_lens[which].copy(), W.n_states, threads=len(which))
    for k, b in enumerate(which):
        np.testing.assert_allclose(loss[:, b].cpu().numpy(), want_loss[:, k], rtol=1e-5, atol=1e-6)
        ref = np.exp(-want_out[:, k].astype(np.float64))
        worst = float(np.abs(post[:, b].cpu().numpy() - ref).max())
        assert worst <= 1e-4, (int(b), worst)


@pytest.mark.parametrize("writer", [-1, 0], ids=["library_choice", "row_writer"])
@pytest.mark.parametrize("layout", ["tbf", "btf"])
def test_more_than_2_to_31_elements(oracle, writer, layout):
    """T*B*F = 2.3e9: element offsets into scores and result do not fit 32 bits from frame 932 on
    (time-major) or from sequence 179 on (batch-major).  Scores are drawn on the device; properties over the whole
    result, the oracle on three sequences (first, middle, last)."""
    B = 192
    W = make_workload("cart", B=B, with_am=False)
    T, F = W.T, W.F
    assert T * B * F > 2 ** 31
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(77)
    am = torch.empty((T, B, F), dtype=torch.float32, device=dev)
    for t0 in range(0, T, 50):
        x = torch.randn((min(50, T - t0), B, F), generator=gen, device=dev) * 3.0
        am[t0:t0 + 50] = -torch.log_softmax(x.double(), -1).float()
    del x
    d = dict(edges=torch.from_numpy(W.edges).to(dev), w=torch.from_numpy(W.weights).to(dev),
             se=torch.from_numpy(W.start_end_states).to(dev), lens=torch.from_numpy(W.seq_lens).to(dev))
    if layout == "tbf":
        out = torch.empty((T, B, F), dtype=torch.float32, device=dev)
        post = out
    else:
        out = torch.empty((B, T, F), dtype=torch.float32, device=dev)
        post = out.transpose(0, 1)
    loss = torch.empty((T, B), dtype=torch.float32, device=dev)
    nbytes = cabi.workspace_size(T, B, F, W.E, W.n_states)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    print(f"2^31: layout {layout} writer {writer} E={W.E} workspace {nbytes >> 20} MiB", flush=True)
    cabi.set_dense_writer(writer)
    try:
        cabi.run_strided(am.data_ptr(), am.stride(0), am.stride(1), 0, d["edges"].data_ptr(), d["edges"].stride(0),
                         d["w"].data_ptr(), d["se"].data_ptr(), d["se"].stride(0), d["lens"].data_ptr(), T, B, F, W.E,
                         W.n_states, cabi.OUT_PROB, out.data_ptr(), post.stride(0), post.stride(1), loss.data_ptr(),
                         ws.data_ptr(), nbytes, stream)
        assert cabi.read_status(ws.data_ptr(), B, stream) == (0, -1)
        assert cabi.last_dense_writer() == (1 if writer < 0 else 0)
    finally:
        cabi.set_dense_writer(-1)
    valid = torch.arange(T, device=dev)[:, None] < d["lens"][None, :]
    rowsum = post.sum(-1, dtype=torch.float64)
    assert torch.all((rowsum[valid] - 1.0).abs() < 1e-4)
    assert torch.all(rowsum[~valid] == 0)
    allowed = torch.zeros((B, F), dtype=torch.bool, device=dev)
    allowed[d["edges"][3].long(), d["edges"][2].long()] = True
    assert torch.all(post.amax(0)[~allowed] == 0)
    first = loss[0][None, :].expand_as(loss)
    assert torch.all(((loss - first).abs() <= 1e-5 * first.abs())[valid])
    _check_sequences_against_oracle(oracle, W, am, post, loss, [0, B // 2, B - 1])


def test_best_path_more_than_2_to_31_elements(oracle):
    """Best path over scores of 2.3e9 elements: alignments and scores of three sequences bit-identical to the oracle's,
    every alignment entry an emission of its sequence."""
    B = 192
    W = make_workload("cart", B=B, with_am=False)
    T, F = W.T, W.F
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(78)
    am = torch.empty((T, B, F), dtype=torch.float32, device=dev)
    for t0 in range(0, T, 50):
        x = torch.randn((min(50, T - t0), B, F), generator=gen, device=dev) * 3.0
        am[t0:t0 + 50] = torch.log_softmax(x.double(), -1).float()
    del x
    d = dict(edges=torch.from_numpy(W.edges).to(dev), w=torch.from_numpy(-W.weights).to(dev),
             se=torch.from_numpy(W.start_end_states).to(dev), lens=torch.from_numpy(W.seq_lens).to(dev))
    align = torch.empty((T, B), dtype=torch.int32, device=dev)
    scores = torch.empty((B,), dtype=torch.float32, device=dev)
    nbytes = cabi.workspace_size(T, B, F, W.E, W.n_states)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    print(f"2^31 best path: E={W.E}", flush=True)
    cabi.viterbi(am.data_ptr(), am.stride(0), am.stride(1), d["edges"].data_ptr(), d["edges"].stride(0), d["w"].data_ptr(),
                 d["se"].data_ptr(), d["se"].stride(0), d["lens"].data_ptr(), T, B, F, W.E, W.n_states,
                 align.data_ptr(), align.stride(0), align.stride(1), scores.data_ptr(), ws.data_ptr(), nbytes, stream)
    assert cabi.read_status(ws.data_ptr(), B, stream) == (0, -1)
    allowed = torch.zeros((B, F), dtype=torch.bool, device=dev)
    allowed[d["edges"][3].long(), d["edges"][2].long()] = True
    valid = torch.arange(T, device=dev)[:, None] < d["lens"][None, :]
    picked = allowed[torch.arange(B, device=dev)[None, :].expand(T, B), align.long().clamp(0, F - 1)]
    assert torch.all(picked[valid])
    which = np.array([0, B // 2, B - 1])
    am_sub = np.ascontiguousarray(am[:, torch.from_numpy(which).to(dev), :].cpu().numpy())
    keep = np.isin(W.edges[3], which)
    edges = W.edges[:, keep].copy()
    edges[3] = np.searchsorted(which, edges[3])
    want_align, want_scores = oracle.viterbi_oracle(am_sub, edges, -W.weights[keep], W.start_end_states[:, which].copy(),
                                                    W.seq_lens[which].copy(), W.n_states)
    np.testing.assert_array_equal(align[:, torch.from_numpy(which).to(dev)].cpu().numpy(), want_align)
    np.testing.assert_array_equal(scores.cpu().numpy()[which].view(np.uint32), want_scores.view(np.uint32))
