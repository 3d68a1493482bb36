"""ctypes view of libi6fbw.so, the C ABI declared in include/i6fbw.h.

Used by the benchmark and the parity tests to call the library exactly as a foreign binding
would: raw device pointers and sizes, caller-owned workspace, caller-chosen stream.  The
PyTorch extension ``fbw_core`` links the same library directly.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "fbw", "libi6fbw.so")

OUT_NEG_LOG = 0
OUT_PROB = 1
OUT_NEG_PROB = 2
IN_LOG_PROBS = 1      # am_scores holds log p instead of -log p
IN_ALL_FRAMES = 2     # gather every (frame, emission) score (needed before an alignment dump)
N_STAGES = 5
STAGE_NAMES = ("prepare", "gather", "recurse", "combine", "padfill")

# every symbol include/i6fbw.h declares
SYMBOLS = ("i6fbw_workspace_size", "i6fbw_run", "i6fbw_run_strided", "i6fbw_read_status", "i6fbw_strerror", "i6fbw_last_hip_error",
           "i6fbw_set_overlap", "i6fbw_viterbi", "i6fbw_dump_output", "i6fbw_dump_alignment",
           "i6fbw_ctc_fsa_bounds", "i6fbw_build_ctc_fsa", "i6fbw_build_hmm_fsa",
           "i6fbw_profile_enable", "i6fbw_profile_read",
           "i6fbw_post_status", "i6fbw_poll_status", "i6fbw_set_status_mode", "i6fbw_get_status_mode",
           "i6fbw_run_static", "i6fbw_static_workspace", "i6fbw_set_dense_writer", "i6fbw_last_dense_writer", "i6fbw_set_spin_limit", "i6fbw_set_band")
STATIC_WORKSPACE_BYTES = 32 << 20
ERR_STATIC_WORKSPACE = -16

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is not built; run `python -m i6_native_ops_amd.build`")
        lib = ctypes.CDLL(LIB_PATH)
        c = ctypes
        lib.i6fbw_workspace_size.argtypes = [c.c_int] * 5 + [c.POINTER(c.c_size_t)]
        lib.i6fbw_workspace_size.restype = c.c_int
        lib.i6fbw_run.argtypes = [c.c_void_p, c.c_int64, c.c_int64, c.c_void_p, c.c_int64, c.c_void_p, c.c_void_p,
                                  c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int,
                                  c.c_void_p, c.c_void_p, c.c_void_p, c.c_size_t, c.c_void_p]
        lib.i6fbw_run.restype = c.c_int
        lib.i6fbw_run_strided.argtypes = [c.c_void_p, c.c_int64, c.c_int64, c.c_int, c.c_void_p, c.c_int64, c.c_void_p,
                                          c.c_void_p, c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int,
                                          c.c_int, c.c_void_p, c.c_int64, c.c_int64, c.c_void_p, c.c_void_p, c.c_size_t,
                                          c.c_void_p]
        lib.i6fbw_run_strided.restype = c.c_int
        lib.i6fbw_run_static.argtypes = [c.c_void_p, c.c_int64, c.c_int64, c.c_void_p, c.c_int64, c.c_void_p, c.c_void_p,
                                         c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int,
                                         c.c_void_p, c.c_void_p, c.c_void_p]
        lib.i6fbw_run_static.restype = c.c_int
        lib.i6fbw_static_workspace.argtypes = [c.POINTER(c.c_void_p), c.POINTER(c.c_size_t)]
        lib.i6fbw_static_workspace.restype = c.c_int
        lib.i6fbw_viterbi.argtypes = [c.c_void_p, c.c_int64, c.c_int64, c.c_void_p, c.c_int64, c.c_void_p, c.c_void_p,
                                      c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int,
                                      c.c_void_p, c.c_int64, c.c_int64, c.c_void_p, c.c_void_p, c.c_size_t, c.c_void_p]
        lib.i6fbw_viterbi.restype = c.c_int
        lib.i6fbw_dump_output.argtypes = [c.c_void_p, c.c_int64, c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_float,
                                          c.c_uint, c.c_char_p, c.c_void_p]
        lib.i6fbw_dump_output.restype = c.c_int
        lib.i6fbw_dump_alignment.argtypes = [c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_void_p, c.c_int64, c.c_float,
                                             c.c_uint, c.c_char_p, c.c_void_p]
        lib.i6fbw_dump_alignment.restype = c.c_int
        lib.i6fbw_ctc_fsa_bounds.argtypes = [c.c_int, c.c_int, c.POINTER(c.c_int), c.POINTER(c.c_int), c.POINTER(c.c_size_t)]
        lib.i6fbw_ctc_fsa_bounds.restype = c.c_int
        lib.i6fbw_build_ctc_fsa.argtypes = [c.c_void_p, c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_void_p, c.c_int64,
                                            c.c_int, c.c_void_p, c.c_void_p, c.c_int64, c.c_void_p, c.c_void_p, c.c_void_p]
        lib.i6fbw_build_ctc_fsa.restype = c.c_int
        lib.i6fbw_build_hmm_fsa.argtypes = [c.c_void_p, c.c_int64, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_void_p, c.c_float,
                                            c.c_float, c.c_void_p, c.c_int64, c.c_int, c.c_void_p, c.c_void_p, c.c_int64,
                                            c.c_void_p, c.c_void_p]
        lib.i6fbw_build_hmm_fsa.restype = c.c_int
        lib.i6fbw_read_status.argtypes = [c.c_void_p, c.c_int, c.c_void_p, c.POINTER(c.c_int), c.POINTER(c.c_int)]
        lib.i6fbw_read_status.restype = c.c_int
        lib.i6fbw_post_status.argtypes = [c.c_void_p, c.c_int, c.c_void_p]
        lib.i6fbw_post_status.restype = c.c_int
        lib.i6fbw_poll_status.argtypes = [c.c_int, c.POINTER(c.c_int), c.POINTER(c.c_int)]
        lib.i6fbw_poll_status.restype = c.c_int
        lib.i6fbw_set_status_mode.argtypes = [c.c_int]
        lib.i6fbw_set_status_mode.restype = None
        lib.i6fbw_get_status_mode.argtypes = []
        lib.i6fbw_get_status_mode.restype = c.c_int
        lib.i6fbw_strerror.argtypes = [c.c_int]
        lib.i6fbw_strerror.restype = c.c_char_p
        lib.i6fbw_last_hip_error.restype = c.c_char_p
        lib.i6fbw_set_overlap.argtypes = [c.c_int]
        lib.i6fbw_set_overlap.restype = None
        lib.i6fbw_set_dense_writer.argtypes = [c.c_int]
        lib.i6fbw_set_dense_writer.restype = None
        lib.i6fbw_set_band.argtypes = [c.c_int]
        lib.i6fbw_set_band.restype = None
        lib.i6fbw_set_spin_limit.argtypes = [c.c_int]
        lib.i6fbw_set_spin_limit.restype = c.c_int
        lib.i6fbw_last_dense_writer.argtypes = []
        lib.i6fbw_last_dense_writer.restype = c.c_int
        lib.i6fbw_profile_enable.argtypes = [c.c_int]
        lib.i6fbw_profile_enable.restype = None
        lib.i6fbw_profile_read.argtypes = [c.POINTER(c.c_float)]
        lib.i6fbw_profile_read.restype = c.c_int
        _lib = lib
    return _lib


class FbwError(RuntimeError):
    def __init__(self, code, seq=None):
        self.code = code
        self.seq = seq
        where = f" (sequence {seq})" if seq is not None and seq >= 0 else ""
        super().__init__(f"i6fbw: {load().i6fbw_strerror(code).decode()}{where}")


def workspace_size(T, B, F, E, n_states) -> int:
    n = ctypes.c_size_t(0)
    rc = load().i6fbw_workspace_size(T, B, F, E, n_states, ctypes.byref(n))
    if rc != 0:
        raise FbwError(rc)
    return int(n.value)


def run(am_ptr, am_stride_t, am_stride_b, edges_ptr, edge_row_stride, weights_ptr, start_end_ptr, se_row_stride,
        seq_lens_ptr, T, B, F, E, n_states, out_mode, out_ptr, sum_ptr, ws_ptr, ws_bytes, stream=0) -> None:
    rc = load().i6fbw_run(am_ptr, am_stride_t, am_stride_b, edges_ptr, edge_row_stride, weights_ptr, start_end_ptr,
                          se_row_stride, seq_lens_ptr, T, B, F, E, n_states, out_mode, out_ptr, sum_ptr, ws_ptr,
                          ws_bytes, stream)
    if rc != 0:
        raise FbwError(rc)


def run_static(am_ptr, am_stride_t, am_stride_b, edges_ptr, edge_row_stride, weights_ptr, start_end_ptr, se_row_stride,
               seq_lens_ptr, T, B, F, E, n_states, out_mode, out_ptr, sum_ptr, stream=0) -> None:
    """i6fbw_run in the library's built-in workspace: allocates nothing."""
    rc = load().i6fbw_run_static(am_ptr, am_stride_t, am_stride_b, edges_ptr, edge_row_stride, weights_ptr, start_end_ptr,
                                 se_row_stride, seq_lens_ptr, T, B, F, E, n_states, out_mode, out_ptr, sum_ptr, stream)
    if rc != 0:
        raise FbwError(rc)


def static_workspace():
    """(device address, bytes) of the current device's built-in workspace."""
    ptr, n = ctypes.c_void_p(0), ctypes.c_size_t(0)
    rc = load().i6fbw_static_workspace(ctypes.byref(ptr), ctypes.byref(n))
    if rc != 0:
        raise FbwError(rc)
    return int(ptr.value), int(n.value)


def run_strided(am_ptr, am_stride_t, am_stride_b, input_flags, edges_ptr, edge_row_stride, weights_ptr,
                start_end_ptr, se_row_stride, seq_lens_ptr, T, B, F, E, n_states, out_mode, out_ptr, out_stride_t,
                out_stride_b, sum_ptr, ws_ptr, ws_bytes, stream=0) -> None:
    rc = load().i6fbw_run_strided(am_ptr, am_stride_t, am_stride_b, int(input_flags), edges_ptr,
                                  edge_row_stride, weights_ptr, start_end_ptr, se_row_stride, seq_lens_ptr, T, B, F, E,
                                  n_states, out_mode, out_ptr, out_stride_t, out_stride_b, sum_ptr, ws_ptr, ws_bytes,
                                  stream)
    if rc != 0:
        raise FbwError(rc)


def viterbi(am_ptr, am_stride_t, am_stride_b, edges_ptr, edge_row_stride, weights_ptr, start_end_ptr, se_row_stride,
            seq_lens_ptr, T, B, F, E, n_states, align_ptr, align_stride_t, align_stride_b, scores_ptr, ws_ptr,
            ws_bytes, stream=0) -> None:
    rc = load().i6fbw_viterbi(am_ptr, am_stride_t, am_stride_b, edges_ptr, edge_row_stride, weights_ptr,
                              start_end_ptr, se_row_stride, seq_lens_ptr, T, B, F, E, n_states, align_ptr,
                              align_stride_t, align_stride_b, scores_ptr, ws_ptr, ws_bytes, stream)
    if rc != 0:
        raise FbwError(rc)


def read_status(ws_ptr, B, stream=0):
    code, seq = ctypes.c_int(0), ctypes.c_int(-1)
    rc = load().i6fbw_read_status(ws_ptr, B, stream, ctypes.byref(code), ctypes.byref(seq))
    if rc != 0:
        raise FbwError(rc)
    return int(code.value), int(seq.value)


def post_status(ws_ptr, B, stream=0):
    """Enqueues the status report of the last call on this workspace; nothing waits."""
    rc = load().i6fbw_post_status(ws_ptr, B, stream)
    if rc != 0:
        raise FbwError(rc)


def poll_status(wait=False):
    """(code, seq) of the first problem among the reports that have arrived (all of them if ``wait``)."""
    code, seq = ctypes.c_int(0), ctypes.c_int(-1)
    rc = load().i6fbw_poll_status(1 if wait else 0, ctypes.byref(code), ctypes.byref(seq))
    if rc != 0:
        raise FbwError(rc)
    return code.value, seq.value


def set_overlap(mode: int) -> None:
    """-1: by problem size, 0: single stream, 1: overlapped stages."""
    load().i6fbw_set_overlap(int(mode))


def set_dense_writer(mode: int) -> None:
    """-1: by problem, 0: row by row, 1: flat spans wherever the output layout allows it."""
    load().i6fbw_set_dense_writer(int(mode))


def set_spin_limit(polls: int) -> None:
    """Polls before a kernel gives up waiting for another kernel of its call (<= 0: the default)."""
    rc = load().i6fbw_set_spin_limit(int(polls))
    if rc != 0:
        raise FbwError(rc)


def last_dense_writer() -> int:
    """0: the last call wrote the tensor row by row, 1: in flat spans."""
    return int(load().i6fbw_last_dense_writer())


def ctc_fsa_bounds(B, Lmax):
    """(edge capacity, state bound, scratch bytes) that always suffice for i6fbw_build_ctc_fsa."""
    e, n, sb = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_size_t(0)
    rc = load().i6fbw_ctc_fsa_bounds(B, Lmax, ctypes.byref(e), ctypes.byref(n), ctypes.byref(sb))
    if rc != 0:
        raise FbwError(rc)
    return int(e.value), int(n.value), int(sb.value)


def build_ctc_fsa(targets_ptr, target_row_stride, target_lens_ptr, B, Lmax, blank, edges_ptr, edge_row_stride, edge_capacity,
                  weights_ptr, start_end_ptr, se_row_stride, totals_ptr, scratch_ptr, stream=0) -> None:
    rc = load().i6fbw_build_ctc_fsa(targets_ptr, target_row_stride, target_lens_ptr, B, Lmax, blank, edges_ptr,
                                    edge_row_stride, edge_capacity, weights_ptr, start_end_ptr, se_row_stride, totals_ptr,
                                    scratch_ptr, stream)
    if rc != 0:
        raise FbwError(rc)


def build_hmm_fsa(labels_ptr, label_row_stride, label_lens_ptr, B, Lmax, states_per_label, emission_table_ptr, loop_weight,
                  forward_weight, edges_ptr, edge_row_stride, edge_capacity, weights_ptr, start_end_ptr, se_row_stride,
                  totals_ptr, stream=0) -> None:
    rc = load().i6fbw_build_hmm_fsa(labels_ptr, label_row_stride, label_lens_ptr, B, Lmax, states_per_label,
                                    emission_table_ptr, loop_weight, forward_weight, edges_ptr, edge_row_stride,
                                    edge_capacity, weights_ptr, start_end_ptr, se_row_stride, totals_ptr, stream)
    if rc != 0:
        raise FbwError(rc)


def dump_alignment(ws_ptr, T, B, E, start_end_ptr, se_row_stride, pruning, batch_idx, directory, stream=0) -> None:
    rc = load().i6fbw_dump_alignment(ws_ptr, T, B, E, start_end_ptr, se_row_stride, pruning, batch_idx,
                                     os.fsencode(directory), stream)
    if rc != 0:
        raise FbwError(rc)


def dump_output(out_ptr, out_stride_t, out_stride_b, seq_lens_ptr, T, B, F, pruning, batch_idx, directory, stream=0) -> None:
    rc = load().i6fbw_dump_output(out_ptr, out_stride_t, out_stride_b, seq_lens_ptr, T, B, F, pruning, batch_idx,
                                  os.fsencode(directory), stream)
    if rc != 0:
        raise FbwError(rc)


def profile_enable(on: bool) -> None:
    load().i6fbw_profile_enable(1 if on else 0)


def profile_read():
    arr = (ctypes.c_float * N_STAGES)()
    n = load().i6fbw_profile_read(arr)
    return n, [float(x) for x in arr]
