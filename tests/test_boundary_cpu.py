"""CPU-side checks of the drop-in boundary: the C ABI library loads and exports every symbol
include/i6fbw.h declares, host-side argument validation, workspace sizing, and the binding's
input checks (no GPU compute)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "i6fbw.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(i6fbw_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from i6_native_ops_amd import cabi
    lib = cabi.load()
    names = declared_symbols()
    assert set(names) == set(cabi.SYMBOLS)
    for n in names:
        assert getattr(lib, n) is not None
    # the in-kernel timestamp hooks (-DI6_TRACE, a measurement build) are not part of the shipped library
    for n in ("i6fbw_debug_trace", "i6fbw_debug_trace_set"):
        assert not hasattr(lib, n), n


def test_workspace_size_and_argument_validation():
    from i6_native_ops_amd import cabi
    n = cabi.workspace_size(1000, 32, 12001, 27000, 12000)
    assert 100e6 < n < 2e9
    assert cabi.workspace_size(50, 2, 10, 60, 32) < n
    for bad in [(0, 1, 1, 1, 1), (1, 0, 1, 1, 1), (1, 1, 0, 1, 1), (1, 1, 1, -1, 1), (1, 1, 1, 1, 0)]:
        with pytest.raises(cabi.FbwError):
            cabi.workspace_size(*bad)
    # null pointers are refused on the host before anything is launched
    with pytest.raises(cabi.FbwError) as e:
        cabi.run(0, 0, 0, 0, 0, 0, 0, 0, 0, 5, 1, 2, 3, 2, 0, 0, 0, 0, 0, 0)
    assert e.value.code == -1
    assert b"invalid" in cabi.load().i6fbw_strerror(-1)
    assert cabi.load().i6fbw_strerror(-12) != cabi.load().i6fbw_strerror(-13)


def test_extension_module_surface():
    import i6_native_ops_amd.fbw as fbw
    assert callable(fbw.fbw_loss) and issubclass(fbw.FastBaumWelchLoss, torch.autograd.Function)
    d = fbw.core.DebugOptions()     # defaults of DebugOptions.h:4-9
    assert (d.dump_alignment, d.dump_output, d.dump_every, d.pruning) == (False, False, 40, 10.0)
    d.dump_every = 7
    assert d.dump_every == 7


def test_binding_rejects_bad_inputs_like_the_reference():
    # CHECK_INPUT (returnn_definitions.h:93-99): device first, then contiguity, then dtype
    import i6_native_ops_amd.fbw as fbw
    am = torch.zeros(5, 1, 2)
    edges = torch.zeros(4, 3, dtype=torch.int32)
    w = torch.zeros(3)
    se = torch.zeros(2, 1, dtype=torch.int32)
    sl = torch.zeros(1, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="am_scores must be a CUDA tensor"):
        fbw.core.fbw(am, edges, w, se, sl, 2)
    with pytest.raises(RuntimeError, match="am_scores must be a CUDA tensor"):
        fbw.core.fbw(am, edges, w, se, sl, 2, fbw.core.DebugOptions())
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        fbw.fbw_loss(torch.zeros(1, 5, 2, requires_grad=True), (2, edges, w, se), sl)


def test_workload_generators_are_deterministic_and_well_formed():
    import numpy as np
    from i6_native_ops_amd.fbw.workloads import WORKLOADS, make_workload
    for name in WORKLOADS:
        a = make_workload(name, with_am=False)
        b = make_workload(name, with_am=False)
        np.testing.assert_array_equal(a.edges, b.edges)
        np.testing.assert_array_equal(a.weights, b.weights)
        assert a.edges.dtype == np.int32 and a.edges.shape[0] == 4
        assert a.edges[:2].max() < a.n_states and a.edges[2].max() < a.F and a.edges[3].max() < a.B
        assert (a.seq_lens >= 1).all() and (a.seq_lens <= a.T).all()
        assert a.algorithmic_bytes() > 4 * a.T * a.B * a.F
    w = make_workload("cart", with_am=False)
    assert (w.T, w.B, w.F) == (1000, 32, 12001)
    per_seq_states = np.diff(np.append(w.start_end_states[0], w.n_states))
    assert per_seq_states.max() <= 451 and per_seq_states.min() >= 301


def test_static_entry_point_refuses_large_problems_on_the_host():
    """i6fbw_run_static checks the size against its built-in workspace before it touches the device."""
    from i6_native_ops_amd import cabi
    import pytest
    with pytest.raises(cabi.FbwError) as e:
        cabi.run_static(256, 32 * 12001, 12001, 256, 30000, 256, 256, 32, 256, 1000, 32, 12001, 30000, 12000, 0, 256, 256, 0)
    assert e.value.code == cabi.ERR_STATIC_WORKSPACE


def test_packaging_metadata():
    """`pip install --no-build-isolation .` is driven by setup.py: its build step is the in-tree build routine
    pointed at the build tree (the install itself compiles for minutes and is not run here)."""
    import ast
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = open(os.path.join(root, "setup.py")).read()
    tree = ast.parse(src)
    names = {n.name for n in ast.walk(tree) if isinstance(n, (ast.ClassDef, ast.FunctionDef))}
    assert {"BuildWithNative", "BinaryDistribution"} <= names
    assert "build_all(os.path.join(self.build_lib" in src
    assert os.path.exists(os.path.join(root, "pyproject.toml"))
    from i6_native_ops_amd import build
    import inspect
    assert "out_root" in inspect.signature(build.build_all).parameters


@pytest.mark.slow
def test_build_step_of_the_install_produces_a_loadable_package(tmp_path):
    """What `pip install --no-build-isolation .` runs (the reference: setup.py:25-64 through torch's BuildExtension):
    setup.py's build step into a scratch build tree, then the C-ABI library of that tree is loaded and exports every
    symbol the header declares, and the tree holds both PyTorch bindings and the version.  Compiles everything:
    minutes."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    build_lib = tmp_path / "lib"
    subprocess.check_call([sys.executable, "setup.py", "-q", "build_py", "--build-lib", str(build_lib)], cwd=root,
                          stdout=subprocess.DEVNULL)
    pkg = build_lib / "i6_native_ops_amd"
    assert (pkg / "fbw" / "libi6fbw.so").exists()
    assert list((pkg / "fbw").glob("fbw_core*.so")) and list((pkg / "fast_viterbi").glob("fast_viterbi_core*.so"))
    # a fresh interpreter that sees the build tree only
    code = ("import sys; sys.path.insert(0, %r); import i6_native_ops_amd; from i6_native_ops_amd import cabi; "
            "assert cabi.__file__.startswith(%r), cabi.__file__; lib = cabi.load(); "
            "missing = [s for s in cabi.SYMBOLS if not hasattr(lib, s)]; assert not missing, missing; "
            "print(i6_native_ops_amd.__version__)") % (str(build_lib), str(build_lib))
    out = subprocess.check_output([sys.executable, "-c", code], cwd=str(tmp_path), text=True)
    from i6_native_ops_amd import __version__
    assert out.strip() == __version__


DENSE_SCRATCH_ALONE = 32      # bytes per lane of fbw_recurse_dense<false>


def test_kernels_stay_within_their_register_budgets():
    """The build records what the compiler reports for every kernel.  The dense writer is launched for eight waves per
    SIMD (64 registers) and the gather, the preparation and the recursion instance for small batches are written to
    need no scratch memory: a change that pushes one of them over its budget makes the compiler spill without a word
    (the dense write of the CTC configuration once went from 0.19 to 0.37 ms that way)."""
    import json
    import os
    from i6_native_ops_amd import cabi
    path = os.path.join(os.path.dirname(cabi.LIB_PATH), "kernel_resources.json")
    if not os.path.exists(path):
        pytest.skip("kernel_resources.json is written by `python -m i6_native_ops_amd.build`")
    res = json.load(open(path))
    # the record belongs to the sources that are here (it is rewritten by every build)
    from i6_native_ops_amd import build
    assert res.get("_sources_sha256") == build.sources_digest(), \
        "kernel_resources.json was made from other kernel sources: rebuild (python -m i6_native_ops_amd.build)"

    def kernels(fragment):
        found = {k: v for k, v in res.items() if fragment in k}
        assert found, fragment
        return found

    for name, r in kernels("fbw_flat").items():
        if name.endswith("Lb1EEEvNS_8FlatArgsE"):      # the instance for the -log output: sums in log space, six waves per SIMD
            assert r["scratch"] == 0 and r["vgprs"] <= 80 and r["occupancy"] >= 6, (name, r)
        else:
            assert r["scratch"] == 0 and r["vgprs"] <= 64 and r["occupancy"] == 8, (name, r)
    for fragment in ("fbw_gather", "fbw_prepare", "fbw_padfill", "fbw_scan_sorted", "11fbw_recurseI", "vit_align"):
        for name, r in kernels(fragment).items():
            assert r["scratch"] == 0, (name, r)
    for name, r in kernels("fbw_recurse_big").items():
        assert r["vgprs"] <= 128 and r["scratch"] == 0, (name, r)          # sixteen waves per compute unit
    for name, r in kernels("fbw_combine").items():
        sync, neglog, small = (int(x) for x in re.search(r"fbw_combineILb(\d)ELb(\d)ELb(\d)E", name).groups())
        if small:
            # the instance for sequences of up to 1024 edges (2048 with short rows): six workgroups per compute unit.
            # Its scratch: values that do not change over a strip of frames, stored once in front of the frame loop
            # and read back once per batch of frames, and a few reloads in the sums of the variant with eight edges
            # per thread (measured: 2.3 times faster than the general instance on such sequences all the same)
            assert r["vgprs"] <= 80 and r["occupancy"] >= 6 and r["scratch"] <= (72 if neglog else 56), (name, r)
        elif neglog:
            # the instance for the -log output: a few reloads per frame on its paths for sequences of more than 1024
            # edges (with two waves per SIMD it needs none and is slower)
            assert r["vgprs"] <= 168 and r["scratch"] <= 124, (name, r)
        else:
            assert r["vgprs"] <= 168 and r["scratch"] == 0, (name, r)      # three waves per SIMD beside a 48 KB row image
    for name, r in kernels("fbw_recurse_dense").items():
        if "ILb0E" in name:
            # stage after stage: two workgroups have a compute unit's registers to themselves; what is left in scratch
            # belongs to the rarely used loop bodies for several states per thread
            assert r["vgprs"] <= 128 and r["scratch"] <= DENSE_SCRATCH_ALONE, (name, r)
        else:
            # beside gather and dense write (a schedule only a test switch selects for such batches): 96 registers, so
            # that their waves find room; the loop bodies for several states per thread pay with spills
            assert r["vgprs"] <= 104 and r["scratch"] <= 264, (name, r)
