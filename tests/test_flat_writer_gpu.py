"""The flat dense writer (fbw_flat: compact posteriors + 128-byte-aligned spans) against the row
writer and the oracle, through the C ABI.

Both writers run the same per-frame arithmetic in the same order, so their outputs must be
identical bit for bit, in every output mode, in both contiguous layouts, at any alignment of the
output tensor, and for batches that mix ordinary sequences with ones the flat kernel leaves to
the row kernel (too large for its posterior jobs), ones whose edges those jobs take in pieces, ones with a reported problem (NaN rows), ones
without edges and ones without frames.
"""
import numpy as np
import pytest

from i6_native_ops_amd.fbw.workloads import make_workload
from tests.helpers import posterior

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
POST_ATOL = 1e-4


def merge(workloads):
    """One batch out of several workloads with the same T and F."""
    T, F = workloads[0].T, workloads[0].F
    edges, weights, se, lens, am = [], [], [], [], []
    s_off = b_off = 0
    for W in workloads:
        assert (W.T, W.F) == (T, F)
        e = W.edges.copy()
        e[0] += s_off
        e[1] += s_off
        e[3] += b_off
        edges.append(e)
        weights.append(W.weights)
        se.append(W.start_end_states + s_off)
        lens.append(W.seq_lens)
        am.append(W.am_scores)
        s_off += W.n_states
        b_off += W.B
    return (np.ascontiguousarray(np.concatenate(am, axis=1)), np.ascontiguousarray(np.concatenate(edges, axis=1)),
            np.concatenate(weights), np.ascontiguousarray(np.concatenate(se, axis=1)), np.concatenate(lens).astype(np.int32), s_off)


def run(args, writer, out_mode, layout, misalign, overlap=1):
    """out (T,B,F) and loss (T,B) as numpy arrays; layout 0: out allocated (T,B,F), 1: (B,T,F);
    misalign: floats between a 256-byte boundary and the start of out"""
    import torch
    from i6_native_ops_amd import cabi
    am, edges, weights, start_end, seq_lens, n_states = args
    T, B, F = am.shape
    E = edges.shape[1]
    dev = torch.device("cuda:0")
    d = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    am_d, edges_d, weights_d, se_d, lens_d = d(am), d(edges), d(weights), d(start_end), d(seq_lens)
    buf = torch.full((T * B * F + 64 + misalign,), -7.0, dtype=torch.float32, device=dev)
    off = (-(buf.data_ptr() // 4) % 64) + misalign
    flat = buf[off:off + T * B * F]
    assert (flat.data_ptr() // 4) % 32 == misalign % 32
    out = flat.view(T, B, F) if layout == 0 else flat.view(B, T, F).transpose(0, 1)
    loss = torch.empty((T, B), dtype=torch.float32, device=dev)
    ws_bytes = cabi.workspace_size(T, B, F, E, n_states)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    cabi.set_overlap(overlap)
    cabi.set_dense_writer(writer)
    try:
        cabi.run_strided(am_d.data_ptr(), am_d.stride(0), am_d.stride(1), 0, edges_d.data_ptr(), edges_d.stride(0) if E else 0,
                         weights_d.data_ptr(), se_d.data_ptr(), se_d.stride(0), lens_d.data_ptr(), T, B, F, E, n_states, out_mode,
                         out.data_ptr(), out.stride(0), out.stride(1), loss.data_ptr(), ws.data_ptr(), ws_bytes, stream)
        code, seq = cabi.read_status(ws.data_ptr(), B, stream)
    finally:
        cabi.set_overlap(-1)
        cabi.set_dense_writer(-1)
    torch.cuda.synchronize()
    # nothing outside the tensor was touched
    assert (buf[:off] == -7.0).all() and (buf[off + T * B * F:] == -7.0).all()
    return out.cpu().numpy(), loss.cpu().numpy(), code, seq


def mixed_batch(T, F, seed):
    """five ordinary sequences, one whose edges the flat kernel's posterior jobs take in two pieces, one too
    large for them (left to the row kernel), and degenerate ones"""
    small = make_workload("cart", seed=seed, T=T, B=8, F=F, n_labels=(4, max(5, T // 12)))
    large = make_workload("cart", seed=seed + 1, T=T, B=1, F=F, n_labels=(180, 180))      # 1080 edges
    large.seq_lens[:] = T
    huge = make_workload("cart", seed=seed + 3, T=T, B=1, F=F, n_labels=(350, 350))       # 2100 edges
    huge.seq_lens[:] = T
    ctc = make_workload("ctc", seed=seed + 2, T=T, B=2, F=F, n_labels=(3, max(4, T // 8)))
    args = list(merge([small, large, ctc, huge]))
    lens = args[4]
    lens[1] = 0                # no frames at all
    lens[2] = T + 5            # out of range: treated like 0 (fbw_op.cu:61-69 never seeds beta)
    lens[3] = 1
    keep = args[1][3] != 4     # sequence 4 loses all of its edges
    args[1] = np.ascontiguousarray(args[1][:, keep])
    args[2] = np.ascontiguousarray(args[2][keep])
    return tuple(args)


@pytest.mark.parametrize("T,F,layout,misalign,out_mode", [
    (70, 128, 0, 0, 0),
    (70, 129, 1, 3, 1),
    (96, 300, 0, 17, 2),
    (64, 517, 1, 0, 0),
    (50, 2048, 0, 31, 1),
    (41, 2500, 1, 8, 1),
    (33, 12001, 0, 5, 0),
    (33, 12001, 1, 0, 2),
    (560, 300, 0, 4, 1),       # long enough for the large sequence (540 states) to carry mass
    (560, 200, 1, 0, 0),
    (600, 2048, 0, 0, 1),      # the same with rows long enough for the flat writer
    (1100, 2050, 1, 6, 0),     # and for the one of 1051 states that is left to the row kernel
])
def test_flat_writer_equals_row_writer_and_oracle(oracle, T, F, layout, misalign, out_mode):
    from i6_native_ops_amd import cabi
    args = mixed_batch(T, F, seed=T + F)
    B = args[0].shape[1]
    out_r, loss_r, code_r, _ = run(args, 0, out_mode, layout, misalign)
    out_f, loss_f, code_f, _ = run(args, 1, out_mode, layout, misalign)
    assert code_r == 0 and code_f == 0
    np.testing.assert_array_equal(loss_f, loss_r)
    np.testing.assert_array_equal(out_f, out_r)
    want_out, want_loss = oracle.fbw_oracle(*args, threads=8)
    want_post = posterior(want_out)
    np.testing.assert_allclose(loss_f, want_loss, rtol=LOSS_RTOL, atol=1e-6)
    got = posterior(out_f) if out_mode == 0 else (out_f if out_mode == 1 else -out_f)
    np.testing.assert_allclose(got, want_post, rtol=0, atol=POST_ATOL)
    hole = np.inf if out_mode == 0 else 0.0
    assert (out_f[np.isposinf(want_out)] == hole).all()


def test_reported_problem_gives_nan_rows_under_both_writers():
    """An emission index out of range in one sequence: its rows below seq_len are NaN, everything else is as without it."""
    from i6_native_ops_amd import cabi
    T, F = 40, 700
    args = list(mixed_batch(T, F, seed=11))
    good = run(tuple(args), 1, 1, 0, 0)
    first = int(np.flatnonzero(args[1][3] == 5)[0])
    args[1] = args[1].copy()
    args[1][2, first] = F                     # sequence 5
    L5 = int(args[4][5])
    for writer in (0, 1):
        out, loss, code, seq = run(tuple(args), writer, 1, 0, 0)
        assert (code, seq) == (-14, 5)
        assert np.isnan(out[:L5, 5]).all() and np.isnan(loss[:L5, 5]).all()
        assert (out[L5:, 5] == 0).all() and (loss[L5:, 5] == 0).all()
        others = [b for b in range(out.shape[1]) if b != 5]
        np.testing.assert_array_equal(out[:, others], good[0][:, others])
        np.testing.assert_array_equal(loss[:, others], good[1][:, others])
    cabi.poll_status(wait=True)


@pytest.mark.parametrize("name", ["cart", "ctc"])
def test_flat_writer_at_scale_equals_row_writer(name):
    """A few hundred megabytes in the layout of fbw_loss: every span, flag and job order of the real grid."""
    W = make_workload(name, T=300 if name == "cart" else 120, B=12 if name == "cart" else 40)
    args = (W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states)
    for layout in (0, 1):
        out_r, loss_r, code_r, _ = run(args, 0, 1, layout, 0)
        out_f, loss_f, code_f, _ = run(args, 1, 1, layout, 0)
        assert code_r == 0 and code_f == 0
        np.testing.assert_array_equal(loss_f, loss_r)
        assert np.array_equal(out_f, out_r)
