"""The overlapped schedule of i6fbw_run under adverse conditions, through the C ABI.

* Another stream keeps the machine busy while an overlapped call is made: the kernels of the call
  wait for each other in memory and need room on the device at the same time; the result must still
  equal the oracle and no wait may run out.
* The give-up path: with the poll limit of the in-memory waits set to 1 from the host, every kernel
  still runs to its normal end, the call reports I6FBW_ERR_TIMEOUT, and every row it could not compute
  holds NaN -- nothing is left uninitialised.
"""
import numpy as np
import pytest

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import posterior

pytestmark = pytest.mark.gpu

ERR_TIMEOUT = -15


def _workload():
    W = make_workload("cart", T=420, B=8, F=3000, n_labels=(30, 45))
    return W, (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)


@pytest.mark.parametrize("writer", [0, 1], ids=["rows", "flat"])
def test_overlapped_call_beside_a_busy_stream(oracle, writer):
    import torch
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    W, args = _workload()
    want_out, want_loss = oracle.fbw_oracle(*args, threads=8)
    P = DeviceProblem(*args)
    side = torch.cuda.Stream()                      # default priority
    x = torch.ones(1 << 27, dtype=torch.float32, device="cuda:0")
    cabi.set_overlap(1)
    cabi.set_dense_writer(writer)
    try:
        for rep in range(3):
            P.out.fill_(-7.0)
            P.loss.fill_(-7.0)
            torch.cuda.synchronize()
            with torch.cuda.stream(side):           # some milliseconds of kernels that fill every compute unit
                for _ in range(12):
                    x.mul_(1.0001).add_(0.5)
            out, loss = P.run(cabi.OUT_PROB)        # raises on any device-side status, a timeout included
            torch.cuda.synchronize()
            np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(out.cpu().numpy(), posterior(want_out), rtol=0, atol=1e-4)
    finally:
        cabi.set_overlap(-1)
        cabi.set_dense_writer(-1)


@pytest.mark.parametrize("writer", [0, 1], ids=["rows", "flat"])
def test_waits_that_run_out_leave_nan_and_a_status(writer):
    import torch
    from i6_native_ops_amd import cabi
    from tests.gpu_util import DeviceProblem
    W, args = _workload()
    P = DeviceProblem(*args)
    good_out, good_loss = P.run(cabi.OUT_PROB)
    good_out, good_loss = good_out.cpu().numpy().copy(), good_loss.cpu().numpy().copy()
    stream = torch.cuda.current_stream().cuda_stream
    cabi.set_overlap(1)
    cabi.set_dense_writer(writer)
    cabi.set_spin_limit(1)
    try:
        P.out.fill_(-7.0)
        P.loss.fill_(-7.0)
        P.run(cabi.OUT_PROB, check=False)
        code, seq = cabi.read_status(P.ws.data_ptr(), P.B, stream)
    finally:
        cabi.set_spin_limit(0)
        cabi.set_overlap(-1)
        cabi.set_dense_writer(-1)
    torch.cuda.synchronize()
    out, loss = P.out.cpu().numpy(), P.loss.cpu().numpy()
    assert code == ERR_TIMEOUT
    # every element was written: NaN where the call gave up, the right value elsewhere
    assert not (out == -7.0).any() and not (loss == -7.0).any()
    bad = np.isnan(out)
    assert bad.any()
    np.testing.assert_array_equal(out[~bad], good_out[~bad])
    lbad = np.isnan(loss)
    np.testing.assert_array_equal(loss[~lbad], good_loss[~lbad])
    for b in range(W.B):                          # rows from seq_len on never depend on a wait
        L = int(W.seq_lens[b])
        assert (out[L:, b] == 0).all() and (loss[L:, b] == 0).all()
    # the next call is unaffected
    out2, loss2 = P.run(cabi.OUT_PROB)
    np.testing.assert_array_equal(out2.cpu().numpy(), good_out)
    np.testing.assert_array_equal(loss2.cpu().numpy(), good_loss)


def test_forced_overlap_with_a_unit_filling_workgroup_per_sequence(oracle):
    """100 chains of 541 states: the recursion instance for large automata, whose workgroups fill a compute
    unit's register file each.  Asked for the overlapped schedule the library declines (200 such workgroups would
    leave the kernels they wait for a fifth of the device, and the waits ran into their bound): the call must
    succeed and equal the oracle either way."""
    from i6_native_ops_amd import cabi
    from tests.gpu_util import run_cabi
    W = make_workload("cart", seed=41, T=640, B=100, F=40, n_labels=(180, 180))
    args = (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    assert W.n_states > 512 * W.B
    want_out, want_loss = oracle.fbw_oracle(*args, threads=16)
    cabi.set_overlap(1)
    try:
        out, loss = run_cabi(*args, out_mode=cabi.OUT_PROB)      # raises on a device-side status
    finally:
        cabi.set_overlap(-1)
    np.testing.assert_allclose(loss, want_loss, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out, posterior(want_out), rtol=0, atol=1e-4)
