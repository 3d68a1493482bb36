"""i6fbw_run_static: the entry point that allocates nothing (built-in workspace).

Checked against i6fbw_run (caller-owned workspace) on the same inputs, through the C ABI: both run
the same kernels in the same order, so the results must be identical bit for bit; on two calls in
a row, the second with a smaller problem (the built-in buffer keeps the first call's contents).
"""
import numpy as np
import pytest

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import random_fsa

pytestmark = pytest.mark.gpu


def _both(args, out_mode):
    import torch
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    p = DeviceProblem(*args)
    want_out, want_loss = p.run(out_mode)
    want_out, want_loss = want_out.cpu().numpy().copy(), want_loss.cpu().numpy().copy()
    p.out.fill_(-7.0)
    p.loss.fill_(-7.0)
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream().cuda_stream
    free_before = torch.cuda.mem_get_info()[0]
    reserved_before = torch.cuda.memory_reserved()
    cabi.run_static(p.am.data_ptr(), p.am.stride(0), p.am.stride(1), p.edges.data_ptr(), p.edges.stride(0) if p.E > 0 else 0,
                    p.weights.data_ptr(), p.start_end.data_ptr(), p.start_end.stride(0), p.seq_lens.data_ptr(), p.T, p.B, p.F,
                    p.E, p.n_states, out_mode, p.out.data_ptr(), p.loss.data_ptr(), stream)
    torch.cuda.synchronize()
    # nothing was allocated: neither by torch nor behind its back (as test/fbw.py:47-55 checks for the reference)
    assert torch.cuda.memory_reserved() == reserved_before
    assert torch.cuda.mem_get_info()[0] == free_before
    ws, nbytes = cabi.static_workspace()
    assert nbytes == cabi.STATIC_WORKSPACE_BYTES and ws % 256 == 0
    code, seq = cabi.read_status(ws, p.B, stream)
    assert code == 0, (code, seq)
    np.testing.assert_array_equal(p.loss.cpu().numpy(), want_loss)
    np.testing.assert_array_equal(p.out.cpu().numpy(), want_out)
    return want_out, want_loss


def _slice(W, T, B):
    """first B sequences and T frames of a workload (lengths cut to T)"""
    keep = W.edges[3] < B
    edges = np.ascontiguousarray(W.edges[:, keep])
    n_states = int(max(edges[:2].max(), W.start_end_states[:, :B].max())) + 1
    return (np.ascontiguousarray(W.am_scores[:T, :B]), edges, np.ascontiguousarray(W.weights[keep]),
            np.ascontiguousarray(W.start_end_states[:, :B]), np.minimum(W.seq_lens[:B], T).astype(np.int32), n_states)


@pytest.mark.parametrize("out_mode", [0, 1])
def test_two_calls_in_a_row_second_smaller(oracle, out_mode):
    from i6_native_ops_amd import cabi
    from tests.helpers import posterior
    W = make_workload("monophone")
    big = _slice(W, 300, 8)            # about 2900 edges: 19 MiB of workspace
    assert cabi.workspace_size(300, 8, W.F, big[1].shape[1], big[5]) <= cabi.STATIC_WORKSPACE_BYTES
    out, loss = _both(big, out_mode)
    # the path under test equals the existing entry point; that one equals the oracle
    want_out, want_loss = oracle.fbw_oracle(*big)
    np.testing.assert_allclose(loss, want_loss, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out if out_mode == 1 else posterior(out), posterior(want_out), rtol=0, atol=1e-4)
    Wt = make_workload("tiny")
    small = (Wt.am_scores, Wt.edges, Wt.weights, Wt.start_end_states, Wt.seq_lens, Wt.n_states)
    out, loss = _both(small, out_mode)
    want_out, want_loss = oracle.fbw_oracle(*small)
    np.testing.assert_allclose(loss, want_loss, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out if out_mode == 1 else posterior(out), posterior(want_out), rtol=0, atol=1e-4)
    # and a third, random one with dead states and parallel edges
    rng = np.random.default_rng(5)
    _both(random_fsa(rng, B=3, F=5, T=7), out_mode)


def test_too_large_is_refused():
    from i6_native_ops_amd import cabi
    W = make_workload("tiny")
    with pytest.raises(cabi.FbwError) as e:
        # sizes only: the call is refused before any pointer is used
        cabi.run_static(256, 32 * 12001, 12001, 256, 30000, 256, 256, 32, 256, 1000, 32, 12001, 30000, 12000, 0, 256, 256, 0)
    assert e.value.code == cabi.ERR_STATIC_WORKSPACE
    assert "32 MiB" in str(e.value)


def test_captured_into_a_graph_and_replayed(oracle):
    """The callers the entry point is for include code under HIP graph capture: the call is captured (after
    i6fbw_static_workspace has set the device up -- kernel attributes and the address of the built-in buffer are taken at
    the first use on a device, which must not fall into a capture), replayed three times with other work of the
    library in between that dirties nothing it owns, and every replay gives what i6fbw_run gives eagerly."""
    import torch
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    W = make_workload("monophone")
    args = _slice(W, 200, 6)
    p = DeviceProblem(*args)
    want_out, want_loss = p.run(cabi.OUT_NEG_LOG)
    want_out, want_loss = want_out.clone(), want_loss.clone()
    cabi.static_workspace()                                 # device set-up outside the capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()

    def call(stream):
        cabi.run_static(p.am.data_ptr(), p.am.stride(0), p.am.stride(1), p.edges.data_ptr(), p.edges.stride(0),
                        p.weights.data_ptr(), p.start_end.data_ptr(), p.start_end.stride(0), p.seq_lens.data_ptr(), p.T, p.B,
                        p.F, p.E, p.n_states, cabi.OUT_NEG_LOG, p.out.data_ptr(), p.loss.data_ptr(), stream)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(side.cuda_stream)
    other = DeviceProblem(*_slice(W, 120, 3))
    for _ in range(3):
        p.out.fill_(-7.0)
        p.loss.fill_(-7.0)
        # another problem through the built-in buffer between the replays: the captured call must not depend on
        # what the buffer held when it was captured
        call_stream = torch.cuda.current_stream().cuda_stream
        cabi.run_static(other.am.data_ptr(), other.am.stride(0), other.am.stride(1), other.edges.data_ptr(), other.edges.stride(0),
                        other.weights.data_ptr(), other.start_end.data_ptr(), other.start_end.stride(0), other.seq_lens.data_ptr(),
                        other.T, other.B, other.F, other.E, other.n_states, cabi.OUT_PROB, other.out.data_ptr(),
                        other.loss.data_ptr(), call_stream)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(p.loss, want_loss)
        assert torch.equal(p.out, want_out)
