"""ctypes front end of the CPU oracle.  TEST INFRASTRUCTURE -- not part of the product.

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  The arithmetic lives in
``fbw_oracle.c`` (a restatement of i6_native_ops/fbw/fbw_op.cu:17-153,226-393) and
``viterbi_oracle.c`` (i6_native_ops/fast_viterbi/core.cu:20-177,209-264).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfbw_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        argt = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,   # am, stride_t, stride_b
            ctypes.c_void_p, ctypes.c_int64,                   # edges, row stride
            ctypes.c_void_p,                                   # weights
            ctypes.c_void_p, ctypes.c_int64,                   # start_end, row stride
            ctypes.c_void_p,                                   # seq_lens
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,  # T B F E n_states
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,    # out, loss, threads
        ]
        for name in ("fbw_oracle_f64", "fbw_oracle_f32"):
            fn = getattr(lib, name)
            fn.argtypes = argt
            fn.restype = ctypes.c_int
        lib.fbw_oracle_max_threads.restype = ctypes.c_int
        lib.viterbi_oracle_f32.argtypes = argt[:-3] + [ctypes.c_void_p, ctypes.c_void_p]
        lib.viterbi_oracle_f32.restype = ctypes.c_int
        _lib = lib
    return _lib


def max_threads() -> int:
    return int(_load().fbw_oracle_max_threads())


def fbw_oracle(am_scores, edges, weights, start_end_states, seq_lens, n_states, precision="f64", threads=1):
    """Same contract as ``fbw_core.fbw`` (fbw_torch.cpp:15-29) on host arrays.

    :param am_scores: float32 [T,B,F], -log probabilities
    :param edges: int32 [4,E] rows from, to, emission_idx, sequence_idx
    :param weights: float32 [E]
    :param start_end_states: int32 [2,B]
    :param seq_lens: int32 [B]
    :return: (out float32 [T,B,F] in -log space with +inf holes, sum_output float64 [T,B])
    """
    lib = _load()
    am = np.ascontiguousarray(am_scores, dtype=np.float32)
    ed = np.ascontiguousarray(edges, dtype=np.int32)
    w = np.ascontiguousarray(weights, dtype=np.float32)
    se = np.ascontiguousarray(start_end_states, dtype=np.int32)
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    T, B, F = am.shape
    assert ed.ndim == 2 and ed.shape[0] == 4
    E = ed.shape[1]
    assert w.shape == (E,) and se.shape == (2, B) and sl.shape == (B,)
    out = np.empty((T, B, F), dtype=np.float32)
    loss = np.empty((T, B), dtype=np.float64)
    fn = lib.fbw_oracle_f64 if precision == "f64" else lib.fbw_oracle_f32
    rc = fn(am.ctypes.data, B * F, F, ed.ctypes.data, E, w.ctypes.data, se.ctypes.data, B, sl.ctypes.data,
            T, B, F, E, int(n_states), out.ctypes.data, loss.ctypes.data, int(threads))
    if rc != 0:
        raise RuntimeError(f"fbw oracle failed with status {rc}")
    return out, loss


def viterbi_oracle(am_scores, edges, weights, start_end_states, seq_lens, n_states):
    """Same contract as ``fast_viterbi_core.fast_viterbi`` (fast_viterbi/binding.cpp:13-25) on host arrays.

    :param am_scores: float32 [T,B,F] scores that are *maximised* (log probabilities)
    :return: (alignment int32 [T,B] of emission indices, 0 in frames without a path; scores float32 [B])
    """
    lib = _load()
    am = np.ascontiguousarray(am_scores, dtype=np.float32)
    ed = np.ascontiguousarray(edges, dtype=np.int32)
    w = np.ascontiguousarray(weights, dtype=np.float32)
    se = np.ascontiguousarray(start_end_states, dtype=np.int32)
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    T, B, F = am.shape
    assert ed.ndim == 2 and ed.shape[0] == 4
    E = ed.shape[1]
    assert w.shape == (E,) and se.shape == (2, B) and sl.shape == (B,)
    alignment = np.empty((T, B), dtype=np.int32)
    scores = np.empty((B,), dtype=np.float32)
    rc = lib.viterbi_oracle_f32(am.ctypes.data, B * F, F, ed.ctypes.data, E, w.ctypes.data, se.ctypes.data, B,
                                sl.ctypes.data, T, B, F, E, int(n_states), alignment.ctypes.data, scores.ctypes.data)
    if rc != 0:
        raise RuntimeError(f"viterbi oracle failed with status {rc}")
    return alignment, scores
