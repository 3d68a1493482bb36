// How the PyTorch bindings hand device-side problems (an index out of range) to Python.  Shared by
// fbw_torch.cpp and viterbi_torch.cpp; the state lives in libi6fbw.so (include/i6fbw.h).
//
//   sync      every call waits for its own result and raises for itself
//   deferred  (default) no call waits: a problem is raised by a later call into the library or by
//             check_status(); the affected sequences hold NaN in the meantime
//   off       never raised
#pragma once
#include <string>

#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include "../../include/i6fbw.h"

namespace i6_status {

inline void report(const char* op, void* workspace, int B, void* stream) {
    const int mode = i6fbw_get_status_mode();
    if (mode == 0) return;
    // while the stream is being captured into a graph nothing may be waited for or queried
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) return;
    int code = 0, seq = -1;
    if (mode == 1) {
        const int rc = i6fbw_read_status(workspace, B, stream, &code, &seq);
        TORCH_CHECK(rc == I6FBW_OK, "NativeOp: ", op, ": ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
        TORCH_CHECK(code == I6FBW_OK, "NativeOp: ", op, ": sequence ", seq, ": ", i6fbw_strerror(code));
        return;
    }
    int rc = i6fbw_post_status(workspace, B, stream);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: ", op, ": ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    rc = i6fbw_poll_status(0, &code, &seq);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: ", op, ": ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    TORCH_CHECK(code == I6FBW_OK, "NativeOp: an earlier call reported: sequence ", seq, ": ", i6fbw_strerror(code));
}

// waits for all reports that are on their way and raises the first problem among them
inline void check_status() {
    int code = 0, seq = -1;
    const int rc = i6fbw_poll_status(1, &code, &seq);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    TORCH_CHECK(code == I6FBW_OK, "NativeOp: an earlier call reported: sequence ", seq, ": ", i6fbw_strerror(code));
}

inline void set_status_mode(const std::string& mode) {
    TORCH_CHECK(mode == "off" || mode == "sync" || mode == "deferred", "status mode must be off, sync or deferred");
    i6fbw_set_status_mode(mode == "off" ? 0 : (mode == "sync" ? 1 : 2));
}

inline std::string get_status_mode() {
    const int mode = i6fbw_get_status_mode();
    return mode == 0 ? "off" : (mode == 1 ? "sync" : "deferred");
}

template <typename Module>
void bind(Module& m) {
    m.def("set_status_mode", &set_status_mode,
          "How device-side problems are raised: 'sync' (by the call itself, which waits for the device), "
          "'deferred' (by a later call or check_status(), no waiting; default), 'off'");
    m.def("get_status_mode", &get_status_mode);
    m.def("check_status", &check_status, "Waits for the calls made so far on this device and raises the first problem they reported");
}

}  // namespace i6_status
