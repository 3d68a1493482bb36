"""The Python front end on the GPU: a port of the reference's own test (test/fbw.py) plus the
behaviours a drop-in has to keep (return shape, ignored grad_loss, fbw_core.fbw contract,
status reporting)."""
import numpy as np
import pytest
import torch

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import posterior, reference_fixture

pytestmark = pytest.mark.gpu


def _fixture_tensors(device="cuda"):
    log_probs = (
        torch.tensor([[0.9, 0.1], [0.9, 0.1], [0.4, 0.6], [0.1, 0.9], [0.1, 0.9]], device=device,
                     dtype=torch.float32, requires_grad=True).unsqueeze(0).log()
    )
    edges = torch.tensor([[0, 0, 0, 0], [0, 1, 0, 0], [1, 1, 1, 0]], device=device,
                         dtype=torch.int32).transpose(0, 1).contiguous()
    weights = torch.tensor([1, 1, 1], device=device, dtype=torch.float32)
    start_end_states = torch.tensor([[0], [1]], dtype=torch.int32, device=device)
    seq_lens = torch.tensor([5], dtype=torch.int32, device=device)
    return log_probs, (2, edges, weights, start_end_states), seq_lens


def test_grad_like_reference_test():
    """test/fbw.py:8-64: no device memory is lost over the call, and -grad sums to 1 per frame."""
    from i6_native_ops_amd.fbw import fbw_loss
    log_probs, fsa, seq_lens = _fixture_tensors()
    log_probs.retain_grad()
    fbw_loss(log_probs.detach(), fsa, seq_lens)       # warm the caching allocator
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    free_pre = torch.cuda.mem_get_info()[0]
    loss = fbw_loss(log_probs, fsa, seq_lens)
    torch.cuda.empty_cache()
    free_post = torch.cuda.mem_get_info()[0]
    # the only memory still held is what the call returned / saved for backward
    held = loss.numel() * 4 + log_probs.numel() * 4 * 2
    assert free_pre - free_post <= max(held, 8 << 20), "memory leak detected in FBW op"
    assert loss.shape == (5, 1)                        # (T, B), not (B,)
    np.testing.assert_allclose(loss.detach().cpu().numpy()[:, 0], 5 - np.log(0.73224), rtol=2e-6)
    loss.sum().backward()
    grad = log_probs.grad
    assert torch.isclose(grad.sum(-1).neg(), torch.full(log_probs.shape[:2], 1.0, device="cuda")).all()


def test_backward_ignores_grad_loss():
    """fbw/__init__.py:40-44 returns the posteriors whatever grad_loss is."""
    from i6_native_ops_amd.fbw import fbw_loss
    grads = []
    for scale in (1.0, 7.0):
        log_probs, fsa, seq_lens = _fixture_tensors()
        log_probs.retain_grad()
        (fbw_loss(log_probs, fsa, seq_lens) * scale).sum().backward()
        grads.append(log_probs.grad.clone())
    assert torch.equal(grads[0], grads[1])


def test_core_fbw_contract(oracle):
    """fbw_core.fbw returns [out (T,B,F) in -log space with +inf holes, sum_output (T,B)]."""
    from i6_native_ops_amd.fbw import core
    W = make_workload("monophone", T=80, B=6, F=60, shuffle_edges=True)
    dev = "cuda"
    out, loss = core.fbw(torch.from_numpy(W.am_scores).to(dev), torch.from_numpy(W.edges).to(dev),
                         torch.from_numpy(W.weights).to(dev), torch.from_numpy(W.start_end_states).to(dev),
                         torch.from_numpy(W.seq_lens).to(dev), W.n_states, core.DebugOptions())
    want_out, want_loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens,
                                            W.n_states)
    assert out.shape == (W.T, W.B, W.F) and loss.shape == (W.T, W.B)
    np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(posterior(out.cpu().numpy()), posterior(want_out), atol=1e-4)
    # holes in exactly the same places, also where a posterior is below float's range: both sides add in log space
    assert (np.isposinf(out.cpu().numpy()) == np.isposinf(want_out)).all()
    # the autograd path yields the same numbers
    from i6_native_ops_amd.fbw import FastBaumWelchLoss
    am = torch.from_numpy(W.am_scores).to(dev).requires_grad_(True)
    fsa = (W.n_states, torch.from_numpy(W.edges).to(dev), torch.from_numpy(W.weights).to(dev),
           torch.from_numpy(W.start_end_states).to(dev))
    l2 = FastBaumWelchLoss.apply(am, fsa, torch.from_numpy(W.seq_lens).to(dev))
    l2.sum().backward()
    # (the posterior mode behind the autograd path adds up the frame normaliser per emission, the -log mode per edge)
    assert torch.all((l2 - loss).abs() <= 1e-6 * loss.abs())
    np.testing.assert_allclose(am.grad.cpu().numpy(), posterior(want_out), atol=1e-4)


def test_non_contiguous_and_wrong_dtype_inputs_raise():
    from i6_native_ops_amd.fbw import core
    log_probs, (n, edges, weights, se), seq_lens = _fixture_tensors()
    am = log_probs.detach().neg().transpose(0, 1).contiguous()
    with pytest.raises(RuntimeError, match="edges must be contiguous"):
        core.fbw(am, edges.t().contiguous().t(), weights, se, seq_lens, n)
    with pytest.raises(RuntimeError, match="Expected seq_lens to contain elements of type"):
        core.fbw(am, edges, weights, se, seq_lens.long(), n)
    with pytest.raises(RuntimeError, match="Expected am_scores to contain elements of type"):
        core.fbw(am.double(), edges, weights, se, seq_lens, n)


def test_device_side_status_is_reported():
    """Indices the reference would read out of bounds with, and automata beyond the supported
    size, surface as RuntimeError instead of the reference's abort()/undefined behaviour."""
    from i6_native_ops_amd.fbw import core
    core.set_status_mode("sync")        # every call waits for its own result (the fixture of conftest.py restores the default)
    log_probs, (n, edges, weights, se), seq_lens = _fixture_tensors()
    am = log_probs.detach().neg().transpose(0, 1).contiguous()
    bad = edges.clone()
    bad[2, 1] = 5                       # emission index >= F
    with pytest.raises(RuntimeError, match="index out of range"):
        core.fbw(am, bad, weights, se, seq_lens, n)
    bad = edges.clone()
    bad[3, 0] = 3                       # sequence index >= B
    with pytest.raises(RuntimeError, match="index out of range"):
        core.fbw(am, bad, weights, se, seq_lens, n)
    # state ids of one sequence spread over far more ids than it has edges: renumbered, same result
    want_out, want_loss = core.fbw(am, edges, weights, se, seq_lens, n)
    sparse = edges.clone()
    sparse[:2][edges[:2] == se[1, 0]] = 40
    out, loss = core.fbw(am, sparse, weights, torch.tensor([[int(se[0, 0])], [40]], dtype=torch.int32, device="cuda"), seq_lens, 41)
    torch.testing.assert_close(loss, want_loss, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(torch.exp(-out), torch.exp(-want_out), rtol=0, atol=1e-5)
    # a state with 9 incoming edges is beyond the fast kernels, not beyond the library
    many = torch.tensor([[0] * 9, [1] * 9, [0] * 9, [0] * 9], dtype=torch.int32, device="cuda")
    out, loss = core.fbw(am, many, torch.zeros(9, device="cuda"), se, torch.tensor([1], dtype=torch.int32, device="cuda"), n)
    assert torch.isfinite(loss[0]).all() and (loss[1:] == 0).all()
    # the good input still works afterwards
    out, loss = core.fbw(am, edges, weights, se, seq_lens, n)
    assert torch.isfinite(loss).all()


@pytest.mark.parametrize("name,kw", [("tiny", {}), ("monophone", dict(T=80, B=6, F=60, shuffle_edges=True)),
                                     ("ctc", dict(T=40, B=8, F=50)), ("cart", dict(T=300, B=3, F=12001))])
@pytest.mark.parametrize("overlap", [0, 1])
def test_fused_fbw_loss_equals_unfused_wrapper_and_oracle(oracle, name, kw, overlap):
    """fbw_loss reads log_probs (B,T,F) in place and writes -posterior in (B,T,F); the reference's
    literal wrapper (neg, transpose, contiguous, exp) must give the same loss and gradient."""
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw import fbw_loss, fbw_loss_unfused
    cabi.set_overlap(overlap)
    try:
        W = make_workload(name, **kw)
        dev = "cuda"
        fsa = (W.n_states, torch.from_numpy(W.edges).to(dev), torch.from_numpy(W.weights).to(dev),
               torch.from_numpy(W.start_end_states).to(dev))
        seq_lens = torch.from_numpy(W.seq_lens).to(dev)
        base = torch.from_numpy(-W.am_scores).transpose(0, 1).contiguous().to(dev)          # [B,T,F] log probs
        results = []
        for fn in (fbw_loss, fbw_loss_unfused):
            lp = base.clone().requires_grad_(True)
            loss = fn(lp, fsa, seq_lens)
            loss.sum().backward()
            results.append((loss.detach().cpu().numpy(), lp.grad.cpu().numpy()))
        want_out, want_loss = oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens,
                                                W.n_states)
        want_grad = -np.exp(-want_out.astype(np.float64)).transpose(1, 0, 2)               # [B,T,F]
        for loss, grad in results:
            assert loss.shape == (W.T, W.B) and grad.shape == (W.B, W.T, W.F)
            np.testing.assert_allclose(loss, want_loss, rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(grad, want_grad, atol=1e-4)
        np.testing.assert_allclose(results[0][0], results[1][0], rtol=1e-6)
        np.testing.assert_allclose(results[0][1], results[1][1], atol=2e-6)
        # a non-contiguous view with unit innermost stride is read in place
        wide = torch.zeros(W.B, W.T, W.F + 5, device=dev)
        wide[:, :, :W.F] = base
        lp = wide[:, :, :W.F].requires_grad_(True)
        loss = fbw_loss(lp, fsa, seq_lens)
        np.testing.assert_array_equal(loss.detach().cpu().numpy(), results[0][0])
    finally:
        cabi.set_overlap(-1)


def test_graph_capture_of_a_large_call(oracle):
    """A call big enough for the overlapped schedule, captured into a HIP graph: the library then
    stays on the capturing stream (no library streams, no in-memory waits, no synchronisation), and
    every replay gives the eager result."""
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    W = make_workload("cart", T=400, B=16, F=12001)            # T*B*F > 2^26
    P = DeviceProblem(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    eager_post, eager_loss = P.run(cabi.OUT_PROB)
    eager_post, eager_loss = eager_post.clone(), eager_loss.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        P.run(cabi.OUT_PROB, check=False)                      # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            P.run(cabi.OUT_PROB, check=False)
    for _ in range(3):
        P.out.fill_(-1.0)
        P.loss.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(P.loss, eager_loss)
        assert torch.equal(P.out, eager_post)


@pytest.mark.parametrize("overlap", [-1, 1], ids=["automatic", "overlapped"])
def test_two_host_threads_on_their_own_streams(overlap):
    """Two threads call the library at the same time, each on its own stream and workspace (the
    library's streams and events are shared by all callers of a device): every call gives the result
    of the same call made alone, bit for bit."""
    import threading
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    workloads = [make_workload("cart", T=400, B=16, F=12001), make_workload("ctc", T=100, B=40, F=300)]
    problems = [DeviceProblem(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states) for W in workloads]
    cabi.set_overlap(overlap)
    try:
        want = []
        for P in problems:
            post, loss = P.run(cabi.OUT_PROB)
            torch.cuda.synchronize()
            want.append((post.clone(), loss.clone()))
        failures = []

        def work(i):
            try:
                P = problems[i]
                stream = torch.cuda.Stream()
                with torch.cuda.stream(stream):
                    for it in range(12):
                        P.loss.fill_(-1.0)
                        post, loss = P.run(cabi.OUT_PROB)
                        stream.synchronize()
                        if not torch.equal(loss, want[i][1]):
                            failures.append((i, it, "loss"))
                    if not torch.equal(post, want[i][0]):
                        failures.append((i, "posteriors"))
            except Exception as exc:        # noqa: BLE001  (reported below, in the main thread)
                failures.append((i, repr(exc)))

        threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not failures, failures
    finally:
        cabi.set_overlap(-1)


def test_deferred_status_does_not_wait_and_is_raised_later():
    """Default mode: a call with an index out of range returns at once, its sequence holds NaN, and the
    problem is raised by check_status() or by the next call that finds the report arrived; after that
    the library is clean again.  Mode 'off' raises nothing."""
    from i6_native_ops_amd.fbw import core
    from i6_native_ops_amd.fast_viterbi import core as vcore
    assert core.get_status_mode() == "deferred" and vcore.get_status_mode() == "deferred"
    log_probs, (n, edges, weights, se), seq_lens = _fixture_tensors()
    am = log_probs.detach().neg().transpose(0, 1).contiguous()
    bad = edges.clone()
    bad[2, 1] = 5                       # emission index >= F
    out, loss = core.fbw(am, bad, weights, se, seq_lens, n)        # no exception here
    assert torch.isnan(loss).all()
    with pytest.raises(RuntimeError, match="an earlier call reported: sequence 0: .*index out of range"):
        core.check_status()
    core.check_status()                 # reported once
    # raised by a later call, of either module, once the report has arrived
    core.fbw(am, bad, weights, se, seq_lens, n)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="an earlier call reported"):
        vcore.fast_viterbi(am, edges, weights, se, seq_lens, n)
    out, loss = core.fbw(am, edges, weights, se, seq_lens, n)
    core.check_status()
    assert torch.isfinite(loss).all()
    # many calls in flight: more than the ring of reports holds
    for _ in range(150):
        core.fbw(am, edges, weights, se, seq_lens, n)
    core.check_status()
    core.set_status_mode("off")
    core.fbw(am, bad, weights, se, seq_lens, n)
    torch.cuda.synchronize()
    core.fbw(am, edges, weights, se, seq_lens, n)
    core.check_status()


@pytest.mark.parametrize("mode", ["deferred", "sync"])
def test_graph_capture_through_the_binding(mode):
    """fbw_loss forward and backward inside torch.cuda.graph: the binding reports no status from a
    capturing stream (nothing there can be waited for or queried), and replays give the eager result."""
    from i6_native_ops_amd.fbw import core, fbw_loss
    core.set_status_mode(mode)
    W = make_workload("cart", T=60, B=4, F=200)
    dev = torch.device("cuda:0")
    fsa = (W.n_states, torch.from_numpy(W.edges).to(dev), torch.from_numpy(W.weights).to(dev),
           torch.from_numpy(W.start_end_states).to(dev))
    seq_lens = torch.from_numpy(W.seq_lens).to(dev)
    static_in = torch.from_numpy(-W.am_scores).transpose(0, 1).contiguous().to(dev).requires_grad_(True)
    eager = fbw_loss(static_in, fsa, seq_lens)
    eager.sum().backward()
    want_loss, want_grad = eager.detach().clone(), static_in.grad.detach().clone()
    del eager                                                # its autograd graph belongs to the default stream
    static_in.grad = None
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):                                   # warm-up on the side stream
            fbw_loss(static_in, fsa, seq_lens).sum().backward()
            static_in.grad = None
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loss = fbw_loss(static_in, fsa, seq_lens)
        loss.sum().backward()
    for _ in range(3):
        loss.fill_(-1.0)
        static_in.grad.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(loss.detach(), want_loss)
        assert torch.equal(static_in.grad, want_grad)
    core.check_status()
