"""DebugOptions text dumps of fbw_core.fbw (fbw_op.cu:155-224,243-247,361-382): file names, line
format, pruning, dump_every, and the values against closed forms on the reference's own fixture."""
import glob
import math
import os

import numpy as np
import pytest
import torch

from tests.helpers import reference_fixture

pytestmark = pytest.mark.gpu


def parse(path):
    rows = []
    for line in open(path):
        t, i, v = line.split()
        rows.append((int(t), int(i), float(v)))
    return rows


def call_fbw(core, fixture, opts):
    am, edges, weights, start_end, seq_lens, n = fixture
    dev = "cuda:0"
    return core.fbw(torch.from_numpy(am).to(dev), torch.from_numpy(edges).to(dev), torch.from_numpy(weights).to(dev),
                    torch.from_numpy(start_end).to(dev), torch.from_numpy(seq_lens).to(dev), n, opts)


@pytest.fixture
def in_tmp(tmp_path):
    old = os.getcwd()
    os.chdir(tmp_path)
    yield tmp_path
    os.chdir(old)


def forward_occupancy():
    """Forward probabilities of the two states of the fixture, frame by frame (the common factor
    exp(-weight) per frame cancels in the normalisation): state 0 loops on label 0, the edge 0->1
    emits label 0, state 1 loops on label 1."""
    e0, e1 = [0.9, 0.9, 0.4, 0.1, 0.1], [0.1, 0.1, 0.6, 0.9, 0.9]
    p = [(1.0, 0.0)]
    for t in range(4):
        p0, p1 = p[-1]
        p.append((p0 * e0[t], p0 * e0[t] + p1 * e1[t]))
    return p


def test_dump_files_on_reference_fixture(in_tmp):
    from i6_native_ops_amd.fbw import core
    opts = core.DebugOptions()
    opts.dump_alignment = True
    opts.dump_output = True
    opts.dump_every = 1
    opts.pruning = 10.0
    call_fbw(core, reference_fixture(), opts)
    torch.cuda.synchronize()
    ali = glob.glob("alignment.dump.*.0")
    tgt = glob.glob("target.dump.*.0")
    assert len(ali) == 1 and len(tgt) == 1
    assert ali[0].split(".")[2] == tgt[0].split(".")[2]            # same batch index

    # alignment: "t state value" with value = -log(forward occupancy of the state)
    got = parse(ali[0])
    want = []
    for t, (p0, p1) in enumerate(forward_occupancy()):
        for s, p in enumerate((p0, p1)):
            if p > 0:
                want.append((t, s, -math.log(p / (p0 + p1))))
    assert [(t, s) for t, s, _ in got] == [(t, s) for t, s, _ in want]
    np.testing.assert_allclose([v for *_, v in got], [v for *_, v in want], atol=2e-5)

    # target: "t emission value" with value = -log posterior (closed form of the five paths)
    post = [[1, 0], [.9402655, .0597345], [.4026549, .5973451], [.0442478, .9557522], [.0044248, .9955752]]
    got = parse(tgt[0])
    want = [(t, e, -math.log(post[t][e])) for t in range(5) for e in range(2) if post[t][e] > 0]
    assert [(t, e) for t, e, _ in got] == [(t, e) for t, e, _ in want]
    np.testing.assert_allclose([v for *_, v in got], [v for *_, v in want], atol=2e-5)


def test_pruning_and_sequence_length(in_tmp):
    from i6_native_ops_amd.fbw import core
    opts = core.DebugOptions()
    opts.dump_alignment = True
    opts.dump_output = True
    opts.dump_every = 1
    opts.pruning = 0.7
    call_fbw(core, reference_fixture(seq_len=4), opts)
    torch.cuda.synchronize()
    for pattern in ("alignment.dump.*.0", "target.dump.*.0"):
        rows = parse(glob.glob(pattern)[0])
        assert rows and all(v <= 0.7 for *_, v in rows)
        assert max(t for t, *_ in rows) <= 3                       # frames >= seq_len are not written
    # occupancies (0.5, 0.5) in frame 1 are 0.6931 <= 0.7: both states listed there
    rows = parse(glob.glob("alignment.dump.*.0")[0])
    assert [(t, s) for t, s, _ in rows if t == 1] == [(1, 0), (1, 1)]


def test_dump_every_and_defaults(in_tmp):
    from i6_native_ops_amd.fbw import core
    # default options: nothing is written
    call_fbw(core, reference_fixture(), core.DebugOptions())
    assert not glob.glob("*.dump.*")
    opts = core.DebugOptions()
    opts.dump_output = True
    opts.dump_every = 2
    for _ in range(4):
        call_fbw(core, reference_fixture(), opts)
    files = sorted(glob.glob("target.dump.*.0"))
    assert len(files) == 2                                         # every second call
    idx = sorted(int(f.split(".")[2]) for f in files)
    assert idx[1] - idx[0] == 2 and idx[0] % 2 == 0
    assert not glob.glob("alignment.dump.*")


def test_process_wide_switch_of_earlier_versions_still_works(in_tmp):
    """i6fbw_set_band(0), the process-wide switch that the per-call flag I6FBW_IN_ALL_FRAMES replaced, is still
    exported for code written against earlier versions of the header: a run under it leaves the same forward rows
    (the same alignment dump) as a run with the flag, and i6fbw_set_band(1) ends it."""
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw.workloads import make_workload
    from tests.gpu_util import DeviceProblem
    wl = make_workload("tiny")
    P = DeviceProblem(wl.am_scores, wl.edges, wl.weights, wl.start_end_states, wl.seq_lens, wl.n_states)
    stream = torch.cuda.current_stream().cuda_stream

    def dump(idx, **kw):
        out, loss = P.run(cabi.OUT_NEG_LOG, **kw)
        cabi.dump_alignment(P.ws.data_ptr(), P.T, P.B, P.E, P.start_end.data_ptr(), P.start_end.stride(0), 1e30, idx, ".", stream)
        return [open(f"alignment.dump.{idx}.{b}").read() for b in range(wl.B)], out.clone(), loss.clone()

    with_flag, out1, loss1 = dump(1, input_flags=cabi.IN_ALL_FRAMES)
    lib = cabi.load()
    lib.i6fbw_set_band(0)
    try:
        with_switch, out2, loss2 = dump(2)
    finally:
        lib.i6fbw_set_band(1)
    banded, out3, loss3 = dump(3)
    assert with_switch == with_flag
    assert torch.equal(out1, out2) and torch.equal(loss1, loss2)
    assert banded != with_flag                    # states that cannot reach the end have no score inside the band
    torch.testing.assert_close(out3, out1, rtol=1e-6, atol=1e-6)


def test_dump_through_the_c_abi(in_tmp, oracle):
    """Two sequences with different lengths straight through i6fbw_dump_*: occupancies of a frame sum to 1,
    the target file lists exactly the finite entries of out."""
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw.workloads import make_workload
    from tests.gpu_util import DeviceProblem
    wl = make_workload("tiny")
    P = DeviceProblem(wl.am_scores, wl.edges, wl.weights, wl.start_end_states, wl.seq_lens, wl.n_states)
    out, _ = P.run(cabi.OUT_NEG_LOG, input_flags=cabi.IN_ALL_FRAMES)
    stream = torch.cuda.current_stream().cuda_stream
    cabi.dump_alignment(P.ws.data_ptr(), P.T, P.B, P.E, P.start_end.data_ptr(), P.start_end.stride(0), 1e30, 7, ".", stream)
    cabi.dump_output(out.data_ptr(), out.stride(0), out.stride(1), P.seq_lens.data_ptr(), P.T, P.B, P.F, 1e30, 7, ".", stream)
    want_out, _ = oracle.fbw_oracle(wl.am_scores, wl.edges, wl.weights, wl.start_end_states, wl.seq_lens, wl.n_states)
    for b in range(wl.B):
        L = int(wl.seq_lens[b])
        rows = parse(f"alignment.dump.7.{b}")
        assert {t for t, *_ in rows} == set(range(L))
        for t in range(L):
            assert sum(math.exp(-v) for tt, _, v in rows if tt == t) == pytest.approx(1.0, abs=1e-4)
        rows = parse(f"target.dump.7.{b}")
        finite = [(t, e) for t in range(L) for e in range(wl.F) if np.isfinite(want_out[t, b, e])]
        assert [(t, e) for t, e, _ in rows] == finite
        np.testing.assert_allclose([v for *_, v in rows], [want_out[t, b, e] for t, e in finite], atol=2e-4, rtol=1e-4)


def _forward_rows(am_b, frm, to, emis, w, start, n_states, L):
    """-log forward scores of every state id before each of the L frames (plain numpy, fbw_op.cu:318-333)"""
    neg = np.full(n_states, -np.inf)
    neg[start] = 0.0
    rows = [-neg]
    for t in range(L - 1):
        cand = neg[frm] - w - am_b[t, emis].astype(np.float64)
        nxt = np.full(n_states, -np.inf)
        np.logaddexp.at(nxt, to, cand)
        neg = nxt
        rows.append(-neg)
    return rows


@pytest.mark.parametrize("case", ["general_path", "spread_ids"])
def test_alignment_dump_of_sequences_off_the_common_path(in_tmp, case):
    """A sequence too large for the fast kernels (more than 8192 edges: general path, rows in double) and one
    whose state ids are spread over a wide range (renumbered on the device): the dump lists the normalised
    forward scores of the ids start..end as for any other sequence (fbw_op.cu:155-196)."""
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw.workloads import make_workload
    from tests.gpu_util import DeviceProblem
    from tests.helpers import spread_state_ids
    if case == "general_path":
        wl = make_workload("cart", T=40, B=2, F=50, n_labels=(1400, 1400))       # 8400 edges per sequence
        edges, start_end, n_states = wl.edges, wl.start_end_states, wl.n_states
    else:
        wl = make_workload("cart", T=40, B=2, F=50, n_labels=(6, 9))
        edges, start_end, n_states = spread_state_ids(wl.edges, wl.start_end_states, wl.n_states, how="stride")
    wl.seq_lens[:] = [40, 33]
    P = DeviceProblem(wl.am_scores, edges, wl.weights, start_end, wl.seq_lens, n_states)
    P.run(cabi.OUT_NEG_LOG, input_flags=cabi.IN_ALL_FRAMES)
    stream = torch.cuda.current_stream().cuda_stream
    pruning = 30.0
    cabi.dump_alignment(P.ws.data_ptr(), P.T, P.B, P.E, P.start_end.data_ptr(), P.start_end.stride(0), pruning, 3, ".", stream)
    for b in range(wl.B):
        L = int(wl.seq_lens[b])
        sel = edges[3] == b
        first, last = int(start_end[0, b]), int(start_end[1, b])
        rows = _forward_rows(wl.am_scores[:, b], edges[0, sel], edges[1, sel], edges[2, sel], wl.weights[sel].astype(np.float64),
                             first, n_states, L)
        got = parse(f"alignment.dump.3.{b}")
        assert {t for t, *_ in got} == set(range(L))
        lo, hi = min(first, last), max(first, last)
        for t in range(L):
            r = rows[t][lo:hi + 1] if first <= last else rows[t][0:0]
            z = -np.logaddexp.reduce(-r)
            want = {i: float(v - z) for i, v in enumerate(r) if v - z <= pruning - 1e-3}
            have = {i: v for tt, i, v in got if tt == t}
            assert set(want) <= set(have)
            for i, v in want.items():
                assert have[i] == pytest.approx(v, abs=2e-4, rel=1e-5)
