/*
 * C ABI of the MI355X (gfx950) full-sum forward-backward (FBW) library, libi6fbw.so.
 *
 * The reference has no C-level interface for this path; its only boundary is
 * the pybind11 function `fbw_core.fbw` (i6_native_ops/fbw/fbw_torch.cpp:15-32)
 * over the CUDA driver `fbw_cuda` (i6_native_ops/fbw/fbw_op.cu:226-393).  The
 * entry points below are what a binding for that function needs: plain
 * pointers and sizes, no torch types.  All data pointers are DEVICE pointers
 * owned by the caller; the library never allocates or frees device memory and
 * never synchronises the device (i6fbw_read_status and i6fbw_poll_status(1, ...) excepted).
 */
#ifndef I6FBW_H
#define I6FBW_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes (return values and i6fbw_read_status). */
enum {
    I6FBW_OK = 0,
    I6FBW_ERR_INVALID_ARGUMENT = -1,   /* null pointer, non-positive T/B/F/n_states, bad out_mode */
    I6FBW_ERR_WORKSPACE_TOO_SMALL = -2,
    I6FBW_ERR_LAUNCH = -3,             /* a HIP launch failed; see i6fbw_last_hip_error() */
    /* Sequences beyond the capacity of the fast kernels (more than 8192 edges, 4096 states or 4096
       distinct emissions in one sequence, more than 15 edges into or out of a state, F beyond
       131 072) are not refused: they take a general path that has no such limits and runs at a
       fraction of the speed. */
    I6FBW_ERR_SEQ_TOO_LARGE = -13,        /* device-side, i6fbw_viterbi only: values and back-pointers of a sequence on the
                                             general path do not fit its share of the workspace (T < 2*edges+16 with
                                             state ids spread over nearly 2*edges ids) */
    I6FBW_ERR_BAD_INDEX = -14,            /* device-side: sequence, emission or state index out of range */
    I6FBW_ERR_TIMEOUT = -15,              /* device-side: a stage gave up waiting for another stage of the call */
    I6FBW_ERR_STATIC_WORKSPACE = -16,     /* i6fbw_run_static: the problem needs more than I6FBW_STATIC_WORKSPACE_BYTES */
    /* Retired: earlier versions of this header refused what the general path now handles.  The names stay so that
       code written against them still compiles; the library never returns these values any more. */
    I6FBW_ERR_F_TOO_LARGE = -4,
    I6FBW_ERR_SEQ_TOO_MANY_EDGES = -10,
    I6FBW_ERR_SEQ_SPARSE_STATES = -11,
    I6FBW_ERR_SEQ_DEGREE = -12
};

/* Layout of the posterior tensor written by i6fbw_run. */
enum {
    I6FBW_OUT_NEG_LOG = 0,   /* -log posterior, +inf where nothing contributes: what fbw_core.fbw returns
                                (fbw_op.cu:366-377,392); finite wherever some edge contributes, however little: the
                                dense write of this mode adds the edges of an emission in log space, as the
                                reference does (fbw_op.cu:39-59,137-153) */
    I6FBW_OUT_PROB = 1,      /* posterior itself, 0 where nothing contributes: what
                                FastBaumWelchLoss.backward derives from it (fbw/__init__.py:40-44) */
    I6FBW_OUT_NEG_PROB = 2   /* minus the posterior: the gradient that reaches `log_probs` in fbw_loss
                                after autograd has undone its neg() (fbw/__init__.py:43,66) */
};

/*
 * Bytes of device workspace i6fbw_run needs for a problem of this size.
 * Replaces the three raw cudaMalloc'ed buffers of fbw_op.cu:283-286.
 */
int i6fbw_workspace_size(int T, int B, int F, int E, int n_states, size_t* bytes);

/*
 * One FBW loss+posterior evaluation; replaces fbw_cuda (fbw_op.cu:226-393)
 * as called from fbw (fbw_torch.cpp:15-29).
 *
 *   am_scores   float [T,B,F], -log probabilities, element strides am_stride_t / am_stride_b,
 *               innermost stride 1                                   (fbw_op.cu:258,268-276)
 *   edges       int32 [4,E] rows from, to, emission_idx, sequence_idx, row stride edge_row_stride
 *                                                                    (fbw_op.cu:249-256)
 *               An edge with sequence_idx -1 is padding and ignored (an extension: the reference
 *               has no such value), so an edge list can be handed over at its capacity.
 *   weights     float [E], -log space                                (fbw_op.cu:257)
 *   start_end   int32 [2,B] row 0 start states, row 1 end states, row stride se_row_stride
 *                                                                    (fbw_op.cu:260-263)
 *   seq_lens    int32 [B]                                            (fbw_op.cu:264)
 *   n_states    number of states of the batch automaton              (fbw_torch.cpp:17)
 *   out         float [T,B,F] contiguous, written completely         (fbw_op.cu:231,265)
 *   sum_output  float [T,B] contiguous: total -log likelihood of sequence b in every frame
 *               t < seq_lens[b], 0 elsewhere                         (fbw_op.cu:104-135,232)
 *   workspace   device buffer of at least i6fbw_workspace_size bytes, 256-byte aligned
 *   stream      hipStream_t to enqueue on (NULL = default stream); the call is asynchronous.
 *               Inside, a large call forks onto library-owned streams (created on first use,
 *               default priority) and joins `stream` again before the call returns, so everything
 *               enqueued on `stream` afterwards sees the finished outputs.  The first large call
 *               on a stream synchronises it once (a check that the library's streams run beside
 *               it); under stream capture the call stays on `stream` and can be replayed.
 *
 * Returns I6FBW_OK or a negative host-side status.  Problems only the device can
 * see (index out of range, an automaton beyond the supported size) are recorded in
 * the workspace and reported by i6fbw_read_status; the affected sequences get NaN
 * in out and sum_output.
 */
int i6fbw_run(const float* am_scores, int64_t am_stride_t, int64_t am_stride_b,
              const int32_t* edges, int64_t edge_row_stride,
              const float* weights,
              const int32_t* start_end, int64_t se_row_stride,
              const int32_t* seq_lens,
              int T, int B, int F, int E, int n_states, int out_mode,
              float* out, float* sum_output,
              void* workspace, size_t workspace_bytes, void* stream);

/*
 * i6fbw_run with explicit layouts, for a caller that holds the (B, T, F) log-probabilities of
 * fbw_loss (fbw/__init__.py:47-68) and wants the gradient in the same layout without the
 * reference wrapper's dense passes (neg, transpose().contiguous(), neg, exp and their autograd
 * inverses: fbw/__init__.py:43,66):
 *   input_flags           I6FBW_IN_LOG_PROBS: am_scores holds log p instead of -log p;
 *                         I6FBW_IN_ALL_FRAMES: gather the score of every (frame, emission) pair, also where
 *                         the emission cannot carry mass (slower, same outputs; i6fbw_dump_alignment needs
 *                         the forward scores of such states).  Per call: nothing process-wide is touched.
 *   out_stride_t/_b       element strides of out over frames / sequences (innermost stride 1);
 *                         rows may overlap nothing else and need not be aligned
 * i6fbw_run(...) is i6fbw_run_strided(..., 0, ..., out, B*F, F, ...).
 */
enum { I6FBW_IN_LOG_PROBS = 1, I6FBW_IN_ALL_FRAMES = 2 };
int i6fbw_run_strided(const float* am_scores, int64_t am_stride_t, int64_t am_stride_b, int input_flags,
                      const int32_t* edges, int64_t edge_row_stride,
                      const float* weights,
                      const int32_t* start_end, int64_t se_row_stride,
                      const int32_t* seq_lens,
                      int T, int B, int F, int E, int n_states, int out_mode,
                      float* out, int64_t out_stride_t, int64_t out_stride_b, float* sum_output,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * i6fbw_run for callers that cannot allocate device memory and therefore have no workspace to
 * bring: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference (whose fbw_cuda allocates and frees three buffers per call,
 * fbw_op.cu:283-286,384-386).  Same arguments and results as i6fbw_run without the workspace: the
 * kernels work in a built-in device buffer of I6FBW_STATIC_WORKSPACE_BYTES that every GPU the
 * library runs on holds until the process ends.  The call allocates nothing (no device or host
 * memory, no streams, no events) and runs all stages one after the other on `stream`.
 * Problems whose workspace (i6fbw_workspace_size) is larger than the built-in buffer are refused
 * with I6FBW_ERR_STATIC_WORKSPACE.  All calls on one GPU share the one buffer: calls that overlap
 * in time on the same GPU (two streams, two host threads) race; calls on one stream are ordered
 * and safe.  i6fbw_static_workspace hands out the buffer of the current device, e.g. for
 * i6fbw_read_status(buffer, B, stream, ...) after a call.  The first use of either function on a device
 * sets kernel attributes and takes the buffer's address there: under graph capture, call
 * i6fbw_static_workspace (or make one eager call) before the capture begins.  The buffer is part of the
 * library's code object: 32 MiB of every GPU the library is used on are taken from the moment it is
 * loaded there, whether or not this entry point is ever called.
 */
#define I6FBW_STATIC_WORKSPACE_BYTES (32u << 20)
int i6fbw_run_static(const float* am_scores, int64_t am_stride_t, int64_t am_stride_b,
                     const int32_t* edges, int64_t edge_row_stride,
                     const float* weights,
                     const int32_t* start_end, int64_t se_row_stride,
                     const int32_t* seq_lens,
                     int T, int B, int F, int E, int n_states, int out_mode,
                     float* out, float* sum_output, void* stream);
int i6fbw_static_workspace(void** workspace, size_t* bytes);

/*
 * Waits for `stream` and copies the device-side status of the last i6fbw_run that
 * used this workspace with batch size B: *code is I6FBW_OK or one of the device-side codes, *seq
 * the first sequence it was seen on.  Replaces the reference's abort()/assert
 * paths (fbw_op.cu:287-290, returnn_definitions.h:114-123) with a status.
 * On a stream that is being captured into a graph nothing can be waited for: the call then
 * reports I6FBW_OK without looking (and i6fbw_post_status enqueues nothing).
 */
int i6fbw_read_status(const void* workspace, int B, void* stream, int* code, int* seq);

/*
 * The same report without a wait, for callers that must not stall the host (a training loop that
 * keeps the device queue full): i6fbw_post_status enqueues, on `stream`, a one-workgroup reduction of
 * the status of the last call that used this workspace with batch size B and its copy into pinned
 * host memory owned by the library (64 reports per device can be in flight; the call waits for the
 * oldest one if all are).  i6fbw_poll_status hands back the first problem among the reports of the
 * current device that have arrived (wait == 0) or among all of them after waiting for them
 * (wait != 0), and forgets it; *code is I6FBW_OK if there is none.  The workspace may be reused or
 * released in stream order after i6fbw_post_status returns.  No counterpart in the reference, whose
 * device-side problems are undefined behaviour (fbw_op.cu:287-290).
 */
int i6fbw_post_status(void* workspace, int B, void* stream);
int i6fbw_poll_status(int wait, int* code, int* seq);

/*
 * How the PyTorch bindings built on this library report device-side problems: 0 not at all, 1 by
 * waiting for every call (i6fbw_read_status; the error belongs to the call that raises it), 2 without
 * waiting (i6fbw_post_status / i6fbw_poll_status; the error is raised by a later call or by the
 * bindings' check_status()).  Initial value: 2, or what the environment variable I6FBW_STATUS
 * (off | sync | deferred) says.
 */
void i6fbw_set_status_mode(int mode);
int i6fbw_get_status_mode(void);

/*
 * Best path (Viterbi alignment) on the same automaton description.  Replaces fast_viterbi_cuda
 * (i6_native_ops/fast_viterbi/core.cu:179-275; binding fast_viterbi/binding.cpp:13-25).
 *
 *   am_scores   float [T,B,F] with element strides am_stride_t / am_stride_b, innermost stride 1;
 *               scores that are MAXIMISED (log probabilities; core.cu:109 adds them to the edge
 *               weight, core.cu:20-49 keeps the larger sum)
 *   edges, weights, start_end, seq_lens, n_states: as for i6fbw_run
 *   alignment   int32, element (t, b) at t * align_stride_t + b * align_stride_b: emission index
 *               of the edge the best path takes in frame t; 0 in frames >= seq_lens[b] and where
 *               the walk back from the end state finds no back-pointer (core.cu:145-177)
 *   scores      float [B]: value of the end state after seq_lens[b] frames, -inf without a path
 *               (core.cu:124-143)
 *   workspace   as for i6fbw_run (i6fbw_workspace_size bytes)
 *
 * Values are computed in the reference's arithmetic, (previous + weight) + score in fp32, and
 * ties go to the edge that comes first in the input, as the reference's compare-and-swap rule
 * decides them, so alignment and scores equal the reference's bit for bit.  seq_lens[b] > T
 * (undefined in the reference) is read as T.  Asynchronous on `stream` (large problems use the
 * library's stream beside it, as i6fbw_run does, and join `stream` before returning); per-sequence
 * problems are reported by i6fbw_read_status, the affected sequences get score NaN and an
 * all-zero alignment.  Sequences beyond the capacity of the fast kernel run the reference's own
 * scheme (per-frame sweeps over the edge list with atomics) and give the same bits.
 */
int i6fbw_viterbi(const float* am_scores, int64_t am_stride_t, int64_t am_stride_b,
                  const int32_t* edges, int64_t edge_row_stride,
                  const float* weights,
                  const int32_t* start_end, int64_t se_row_stride,
                  const int32_t* seq_lens,
                  int T, int B, int F, int E, int n_states,
                  int32_t* alignment, int64_t align_stride_t, int64_t align_stride_b, float* scores,
                  void* workspace, size_t workspace_bytes, void* stream);

/*
 * Chooses how i6fbw_run schedules its stages: 0 one after the other on the caller's stream,
 * 1 overlapped (gather, recursion and dense write run at the same time on library streams and
 * hand frames to each other through flags in the workspace), -1 (default) overlapped for large
 * problems only.  The environment variable I6FBW_OVERLAP=0/1 sets the initial value.  Results do
 * not depend on the schedule.  No counterpart in the reference.
 */
void i6fbw_set_overlap(int mode);

/*
 * DEPRECATED, kept so that code written against earlier versions of this header still builds and behaves:
 * i6fbw_set_band(0) makes every later call of the process run as if it had been given I6FBW_IN_ALL_FRAMES,
 * i6fbw_set_band(1) (the default) ends that.  New code passes the flag to the one call that needs it
 * (i6fbw_run_strided).  No counterpart in the reference.
 */
void i6fbw_set_band(int on);

/*
 * TEST HOOK, not for production code.  Kernels of the overlapped schedule that wait for another kernel
 * of the same call poll at most `polls` times (default 2^20, restored by polls <= 0) before they give up:
 * the call then reports I6FBW_ERR_TIMEOUT and the rows that could not be computed hold NaN.  It exists so
 * that a test can force that path from the host (polls = 1) while every kernel still runs to its normal
 * end.  Device-wide for the current device: the call waits for the device to go idle, takes the lock that
 * serialises the library's calls on it, and changes the limit for every call enqueued afterwards by any
 * thread -- a thread that calls i6fbw_run on the same device at the same time gets either limit.
 * No counterpart in the reference.
 */
int i6fbw_set_spin_limit(int polls);

/*
 * Chooses how i6fbw_run writes the dense (T, B, F) tensor: 0 row by row (one workgroup per strip of
 * frames of a sequence builds each row in LDS and streams it out), 1 in flat 128-byte-aligned spans
 * fed from compact per-frame posteriors wherever the output is one contiguous block ((T, B, F) or
 * (B, T, F) order, F >= 128), -1 (default) flat spans for the large problems whose stages overlap.
 * The environment variable I6FBW_DENSE_WRITER=rows|flat sets the initial value.  Results do not
 * depend on the writer.  No counterpart in the reference (fbw_op.cu:137-153,366-377 scatter with
 * atomics into a pre-filled tensor).
 */
void i6fbw_set_dense_writer(int mode);
/* Which writer the most recent i6fbw_run / i6fbw_run_strided of the process used: 0 rows, 1 flat spans
 * (for benchmarks that price the kernel that wrote the tensor). */
int i6fbw_last_dense_writer(void);

/*
 * Device-side construction of the automaton arrays for two common topologies.  No counterpart in
 * the reference, which leaves the tuple (number of states, edges, weights, start/end states) to
 * its callers (fbw/__init__.py:56-62); these take that step off the host.  States of sequence b
 * are contiguous and follow those of sequence b-1, edges are grouped by sequence.  Edges from the
 * number actually produced up to edge_capacity are written as padding edges (sequence index -1),
 * which i6fbw_run and i6fbw_viterbi skip: pass E = edge_capacity and any upper bound of the number
 * of states as n_states, and the host never needs the exact counts.  totals (device, 2 ints)
 * receives them anyway: [0] edges produced, [1] states.
 *
 * i6fbw_build_ctc_fsa: CTC with the emission on the target state of an edge.  Per sequence with
 * labels l_1..l_L (targets[b * target_row_stride + i], L = target_lens[b] limited to [0, Lmax]): a
 * non-emitting start state, the 2L+1 states blank, l_1, blank, ..., l_L, blank and a terminal end
 * state; loops, edges to the next state, label-to-next-label edges where the labels differ, the
 * start state feeding the first blank and the first label, and a copy into the terminal state of
 * every edge that enters the last label or the last blank.  All weights 0.  With these arrays
 * i6fbw_run's sum_output equals torch.nn.functional.ctc_loss(reduction="none") per sequence.
 * i6fbw_ctc_fsa_bounds gives capacities that always suffice and the size of `scratch` (device).
 *
 * i6fbw_build_hmm_fsa: left-to-right chain, states_per_label states per label, each with a loop
 * (loop_weight) and an edge to the next state (forward_weight), both emitting
 * emission_table[label * states_per_label + k] (the index itself if emission_table is NULL): the
 * emission sits on the source state as in the reference's test (test/fbw.py:28-32); the last state
 * leads to a non-emitting end state.  Exactly 2 * states_per_label * sum(L) edges and
 * states_per_label * sum(L) + B states; capacities B * Lmax * states_per_label * 2 and
 * B * (Lmax * states_per_label + 1) always suffice.  totals may be NULL if edge_capacity is exact.
 */
int i6fbw_ctc_fsa_bounds(int B, int Lmax, int* max_edges, int* max_states, size_t* scratch_bytes);
int i6fbw_build_ctc_fsa(const int32_t* targets, int64_t target_row_stride, const int32_t* target_lens, int B, int Lmax,
                        int blank, int32_t* edges, int64_t edge_row_stride, int edge_capacity, float* weights,
                        int32_t* start_end, int64_t se_row_stride, int32_t* totals, void* scratch, void* stream);
int i6fbw_build_hmm_fsa(const int32_t* labels, int64_t label_row_stride, const int32_t* label_lens, int B, int Lmax,
                        int states_per_label, const int32_t* emission_table, float loop_weight, float forward_weight,
                        int32_t* edges, int64_t edge_row_stride, int edge_capacity, float* weights,
                        int32_t* start_end, int64_t se_row_stride, int32_t* totals, void* stream);

/*
 * Debug dumps of the reference (fbw_op.cu:155-224, switched by DebugOptions, DebugOptions.h:4-9).
 * Host-side helpers: they synchronise `stream`, copy to the host and write one text file per
 * sequence into `directory` (the reference writes into the working directory).
 *
 * i6fbw_dump_output: file target.dump.<batch_idx>.<seq>, a line "t e value" for every element of
 * out[t, seq, :] (as written with I6FBW_OUT_NEG_LOG) that is <= pruning, for t < seq_lens[seq]
 * (frame 0 always), as write_output_to_file (fbw_op.cu:199-224).
 *
 * i6fbw_dump_alignment: file alignment.dump.<batch_idx>.<seq>, a line "t (state - start) value"
 * for the states start..end of the sequence, where value = forward score of the state before
 * frame t minus the log-sum over those states, if <= pruning, as write_alignment_to_file
 * (fbw_op.cu:155-197).  It reads the forward rows of the last i6fbw_run_strided on `workspace`; make
 * that call with I6FBW_IN_ALL_FRAMES, otherwise states that cannot reach the end state in the
 * remaining frames are missing (their scores are never computed).
 * Sequences whose length is outside [1, T] have no forward rows: frame 0 alone is written.
 */
int i6fbw_dump_output(const float* out, int64_t out_stride_t, int64_t out_stride_b, const int32_t* seq_lens,
                      int T, int B, int F, float pruning, unsigned batch_idx, const char* directory, void* stream);
int i6fbw_dump_alignment(const void* workspace, int T, int B, int E, const int32_t* start_end, int64_t se_row_stride,
                         float pruning, unsigned batch_idx, const char* directory, void* stream);

/* Text for a status code. */
const char* i6fbw_strerror(int code);

/* hipGetErrorString of the last failed HIP call of this thread ("" if none). */
const char* i6fbw_last_hip_error(void);

/*
 * Average device time per call, in milliseconds, of each stage over all i6fbw_run calls since
 * profiling was switched on, measured with HIP event pairs around every launch of the stage on
 * the stream that launch runs on (the stages of one call overlap in time, so the entries do not
 * add up to the call's duration).  Off by default; i6fbw_profile_enable(1) turns it on and clears
 * the sums, i6fbw_profile_enable(0) turns it off.  stage_ms has room for I6FBW_N_STAGES entries:
 * 0 edge preparation, 1 emission gather, 2 alpha/beta recursion, 3 combine + dense write of the
 * frames that carry probability mass, 4 fill of the remaining rows.  Keeps at most 8192 launches.
 * i6fbw_profile_read waits for the recorded events, returns the number of calls averaged over
 * and clears the sums.
 */
#define I6FBW_N_STAGES 5
void i6fbw_profile_enable(int on);
int i6fbw_profile_read(float* stage_ms);

#ifdef __cplusplus
}
#endif
#endif /* I6FBW_H */
