// PyTorch-ROCm binding of libi6fbw.so: module `fbw_core` with the reference's interface
// (i6_native_ops/fbw/fbw_torch.cpp:15-40): fbw(am_scores, edges, weights, start_end_states,
// seq_lens, num_states, debug_options=DebugOptions()) -> [out (T,B,F), sum_output (T,B)].
// torch is used for device memory and the current stream only; all arithmetic is behind the
// C ABI declared in include/i6fbw.h.
#include <atomic>
#include <cstdlib>
#include <vector>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include "../../include/i6fbw.h"
#include "status_report.h"

namespace py = pybind11;

// Same fields and defaults as the reference's DebugOptions.h:4-9.
struct DebugOptions {
    bool dump_alignment = false;
    bool dump_output = false;
    unsigned dump_every = 40u;
    float pruning = 10.f;
};

// Same checks and messages as CHECK_INPUT (common/returnn_definitions.h:93-99).
#define CHECK_CUDA(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_TYPE(x, type) \
    TORCH_CHECK(x.dtype() == type, "Expected " #x " to contain elements of type ", type, ", but got type ", x.dtype())
#define CHECK_INPUT(x, type) \
    CHECK_CUDA(x);           \
    CHECK_CONTIGUOUS(x);     \
    CHECK_TYPE(x, type)

// fused == false: am_scores is (T, B, F), -log p, contiguous; out is (T, B, F).
// fused == true:  am_scores is log_probs (B, T, F) with unit innermost stride; out is (B, T, F).
static std::vector<torch::Tensor> run(torch::Tensor& am_scores, torch::Tensor& edges, torch::Tensor& weights,
                                      torch::Tensor& start_end_states, torch::Tensor& seq_lens, unsigned num_states,
                                      int out_mode, bool fused = false, const DebugOptions* dump = nullptr,
                                      unsigned batch_idx = 0u) {
    if (fused) {
        CHECK_CUDA(am_scores);
        CHECK_TYPE(am_scores, torch::kFloat32);
        TORCH_CHECK(am_scores.dim() == 3 && am_scores.stride(2) == 1, "log_probs must have shape (B, T, F) with unit innermost stride");
    } else {
        CHECK_INPUT(am_scores, torch::kFloat32);
    }
    CHECK_INPUT(edges, torch::kInt32);
    CHECK_INPUT(weights, torch::kFloat32);
    CHECK_INPUT(start_end_states, torch::kInt32);
    CHECK_INPUT(seq_lens, torch::kInt32);
    // shape relations the reference asserts (fbw_op.cu:234-241,278-279)
    TORCH_CHECK(am_scores.dim() == 3, "am_scores must have shape (T, B, F)");
    const int dt = fused ? 1 : 0, db = fused ? 0 : 1;      // which dimension is time / batch
    TORCH_CHECK(edges.dim() == 2 && edges.size(0) == 4, "edges must have shape (4, E)");
    TORCH_CHECK(weights.dim() == 1 && weights.size(0) == edges.size(1), "weights must have shape (E,)");
    TORCH_CHECK(start_end_states.dim() == 2 && start_end_states.size(0) == 2 &&
                    start_end_states.size(1) == am_scores.size(db),
                "start_end_states must have shape (2, B)");
    TORCH_CHECK(seq_lens.dim() == 1 && seq_lens.size(0) == am_scores.size(db), "seq_lens must have shape (B,)");
    TORCH_CHECK(am_scores.size(0) > 0 && am_scores.size(1) > 0 && am_scores.size(2) > 0 && num_states > 0,
                "NativeOp assertion failed: n_frames > 0, n_states > 0");
    const int T = (int)am_scores.size(dt), B = (int)am_scores.size(db), F = (int)am_scores.size(2);
    const int E = (int)edges.size(1);

    // PyTorch-ROCm presents HIP devices under the device type "cuda"
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(am_scores.device());
    auto opts = torch::TensorOptions().device(am_scores.device());
    torch::Tensor out = torch::empty(am_scores.sizes(), opts.dtype(torch::kFloat32));      // contiguous, same shape
    torch::Tensor sum_output = torch::empty({T, B}, opts.dtype(torch::kFloat32));
    size_t ws_bytes = 0;
    int rc = i6fbw_workspace_size(T, B, F, E, (int)num_states, &ws_bytes);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fbw: ", i6fbw_strerror(rc));
    torch::Tensor workspace = torch::empty({(int64_t)ws_bytes}, opts.dtype(torch::kUInt8));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    // the alignment dump needs the forward scores of every state, also of those that cannot reach
    // the end state any more
    const bool all_scores = dump && dump->dump_alignment;
    const int input_flags = (fused ? I6FBW_IN_LOG_PROBS : 0) | (all_scores ? I6FBW_IN_ALL_FRAMES : 0);
    rc = i6fbw_run_strided(am_scores.data_ptr<float>(), am_scores.stride(dt), am_scores.stride(db), input_flags,
                           edges.data_ptr<int32_t>(), edges.stride(0), weights.data_ptr<float>(),
                           start_end_states.data_ptr<int32_t>(), start_end_states.stride(0),
                           seq_lens.data_ptr<int32_t>(), T, B, F, E, (int)num_states, out_mode, out.data_ptr<float>(),
                           out.stride(dt), out.stride(db), sum_output.data_ptr<float>(), workspace.data_ptr(), ws_bytes,
                           (void*)stream);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fbw: ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    // a dump reads the workspace on the host anyway: such a call waits for its own status
    if (dump && i6fbw_get_status_mode() == 2) {
        int code = 0, seq = -1;
        rc = i6fbw_read_status(workspace.data_ptr(), B, (void*)stream, &code, &seq);
        TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fbw: ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
        TORCH_CHECK(code == I6FBW_OK, "NativeOp: fbw: sequence ", seq, ": ", i6fbw_strerror(code));
    } else {
        i6_status::report("fbw", workspace.data_ptr(), B, (void*)stream);
    }
    if (dump && dump->dump_alignment) {
        // as fbw_op.cu:361-364
        rc = i6fbw_dump_alignment(workspace.data_ptr(), T, B, E, start_end_states.data_ptr<int32_t>(),
                                  start_end_states.stride(0), dump->pruning, batch_idx, ".", (void*)stream);
        TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fbw: alignment dump: ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    }
    if (dump && dump->dump_output) {
        // as fbw_op.cu:379-381
        rc = i6fbw_dump_output(out.data_ptr<float>(), out.stride(dt), out.stride(db), seq_lens.data_ptr<int32_t>(), T, B, F,
                               dump->pruning, batch_idx, ".", (void*)stream);
        TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fbw: output dump: ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    }
    return {out, sum_output};
}

std::vector<torch::Tensor> fbw(torch::Tensor& am_scores, torch::Tensor& edges, torch::Tensor& weights,
                               torch::Tensor& start_end_states, torch::Tensor& seq_lens, unsigned num_states,
                               DebugOptions debug_options = DebugOptions()) {
    // calls are numbered as in the reference (fbw_op.cu:246,390); every dump_every-th one is dumped
    static std::atomic<unsigned> batch_idx{0u};
    const unsigned idx = batch_idx++;
    const bool dump_now = (debug_options.dump_alignment || debug_options.dump_output) && debug_options.dump_every > 0u &&
                          idx % debug_options.dump_every == 0u;
    return run(am_scores, edges, weights, start_end_states, seq_lens, num_states, I6FBW_OUT_NEG_LOG, false,
               dump_now ? &debug_options : nullptr, idx);
}

std::vector<torch::Tensor> fbw_posterior(torch::Tensor& am_scores, torch::Tensor& edges, torch::Tensor& weights,
                                         torch::Tensor& start_end_states, torch::Tensor& seq_lens,
                                         unsigned num_states) {
    return run(am_scores, edges, weights, start_end_states, seq_lens, num_states, I6FBW_OUT_PROB);
}

// The whole of fbw_loss in one call: log_probs (B, T, F) in, [-posterior (B, T, F), loss (T, B)] out.
// -posterior is what autograd delivers to log_probs through the reference wrapper's
// neg().transpose(0, 1).contiguous() (fbw/__init__.py:66) and backward (fbw/__init__.py:40-44).
std::vector<torch::Tensor> fbw_fused(torch::Tensor& log_probs, torch::Tensor& edges, torch::Tensor& weights,
                                     torch::Tensor& start_end_states, torch::Tensor& seq_lens, unsigned num_states) {
    return run(log_probs, edges, weights, start_end_states, seq_lens, num_states, I6FBW_OUT_NEG_PROB, true);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    py::class_<DebugOptions>(m, "DebugOptions")
        .def(py::init<>())
        .def_readwrite("dump_alignment", &DebugOptions::dump_alignment)
        .def_readwrite("dump_output", &DebugOptions::dump_output)
        .def_readwrite("dump_every", &DebugOptions::dump_every)
        .def_readwrite("pruning", &DebugOptions::pruning);

    m.def("fbw", &fbw, "Fast Baum-Welch routine (MI355X)", py::arg("am_scores"), py::arg("edges"), py::arg("weights"),
          py::arg("start_end_states"), py::arg("seq_lens"), py::arg("num_states"),
          py::arg("debug_options") = DebugOptions());
    m.def("fbw_fused", &fbw_fused,
          "fbw_loss in one call: log_probs (B, T, F) -> [gradient w.r.t. log_probs = -posterior (B, T, F), loss (T, B)]");
    i6_status::bind(m);
    m.def("fbw_posterior", &fbw_posterior,
          "Same as fbw but the first result holds the posteriors themselves (exp(-out)) with 0 in the holes");
}
