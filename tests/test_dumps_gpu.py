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


def test_dump_through_the_c_abi(in_tmp, oracle):
    """Two sequences with different lengths straight through i6fbw_dump_*: occupancies of a frame sum to 1,
    the target file lists exactly the finite entries of out."""
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw.workloads import make_workload
    from tests.gpu_util import DeviceProblem
    wl = make_workload("tiny")
    cabi.set_band(False)
    try:
        P = DeviceProblem(wl.am_scores, wl.edges, wl.weights, wl.start_end_states, wl.seq_lens, wl.n_states)
        out, _ = P.run(cabi.OUT_NEG_LOG)
    finally:
        cabi.set_band(True)
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
