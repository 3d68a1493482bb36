// PyTorch-ROCm binding of the best-path search in libi6fbw.so: module `fast_viterbi_core` with the
// reference's interface (i6_native_ops/fast_viterbi/binding.cpp:13-29):
// fast_viterbi(am_scores, edges, weights, start_end_states, seq_lens, num_states) -> [alignment (T,B) int32, scores (B,)].
// torch is used for device memory and the current stream only.
#include <cstdlib>
#include <vector>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include "../../include/i6fbw.h"
#include "status_report.h"

// Same checks and messages as CHECK_INPUT (common/returnn_definitions.h:93-99).
#define CHECK_CUDA(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_TYPE(x, type) \
    TORCH_CHECK(x.dtype() == type, "Expected " #x " to contain elements of type ", type, ", but got type ", x.dtype())
#define CHECK_INPUT(x, type) \
    CHECK_CUDA(x);           \
    CHECK_CONTIGUOUS(x);     \
    CHECK_TYPE(x, type)

// batch_major == false: am_scores is (T, B, F) contiguous, alignment comes back as (T, B).
// batch_major == true:  am_scores is (B, T, F) with unit innermost stride, alignment comes back as (B, T).
static std::vector<torch::Tensor> run(torch::Tensor& am_scores, torch::Tensor& edges, torch::Tensor& weights,
                                      torch::Tensor& start_end_states, torch::Tensor& seq_lens, unsigned num_states,
                                      bool batch_major) {
    if (batch_major) {
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
    // shape relations the reference asserts (fast_viterbi/core.cu:184-201)
    TORCH_CHECK(am_scores.dim() == 3, "am_scores must have shape (T, B, F)");
    const int dt = batch_major ? 1 : 0, db = batch_major ? 0 : 1;
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

    const c10::hip::HIPGuardMasqueradingAsCUDA guard(am_scores.device());
    auto opts = torch::TensorOptions().device(am_scores.device());
    torch::Tensor alignment = batch_major ? torch::empty({B, T}, opts.dtype(torch::kInt32))
                                          : torch::empty({T, B}, opts.dtype(torch::kInt32));
    torch::Tensor scores = torch::empty({B}, opts.dtype(torch::kFloat32));
    size_t ws_bytes = 0;
    int rc = i6fbw_workspace_size(T, B, F, E, (int)num_states, &ws_bytes);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fast_viterbi: ", i6fbw_strerror(rc));
    torch::Tensor workspace = torch::empty({(int64_t)ws_bytes}, opts.dtype(torch::kUInt8));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    rc = i6fbw_viterbi(am_scores.data_ptr<float>(), am_scores.stride(dt), am_scores.stride(db),
                       edges.data_ptr<int32_t>(), edges.stride(0), weights.data_ptr<float>(),
                       start_end_states.data_ptr<int32_t>(), start_end_states.stride(0), seq_lens.data_ptr<int32_t>(),
                       T, B, F, E, (int)num_states, alignment.data_ptr<int32_t>(), alignment.stride(dt),
                       alignment.stride(db), scores.data_ptr<float>(), workspace.data_ptr(), ws_bytes, (void*)stream);
    TORCH_CHECK(rc == I6FBW_OK, "NativeOp: fast_viterbi: ", i6fbw_strerror(rc), " ", i6fbw_last_hip_error());
    i6_status::report("fast_viterbi", workspace.data_ptr(), B, (void*)stream);
    return {alignment, scores};
}

std::vector<torch::Tensor> fast_viterbi(torch::Tensor& am_scores, torch::Tensor& edges, torch::Tensor& weights,
                                        torch::Tensor& start_end_states, torch::Tensor& seq_lens, unsigned num_states) {
    return run(am_scores, edges, weights, start_end_states, seq_lens, num_states, false);
}

// align_viterbi in one call: log_probs (B, T, F) read in place, alignment written as (B, T), without the
// wrapper's transpose().contiguous() passes (fast_viterbi/__init__.py:40,46).
std::vector<torch::Tensor> fast_viterbi_batch_major(torch::Tensor& log_probs, torch::Tensor& edges, torch::Tensor& weights,
                                                    torch::Tensor& start_end_states, torch::Tensor& seq_lens,
                                                    unsigned num_states) {
    return run(log_probs, edges, weights, start_end_states, seq_lens, num_states, true);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("fast_viterbi", &fast_viterbi, "Fast Viterbi routine (MI355X)");
    i6_status::bind(m);
    m.def("fast_viterbi_batch_major", &fast_viterbi_batch_major,
          "align_viterbi in one call: log_probs (B, T, F) -> [alignment (B, T) int32, scores (B,)]");
}
