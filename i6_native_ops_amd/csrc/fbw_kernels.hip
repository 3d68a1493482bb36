// Full-sum forward-backward (FBW) loss for MI355X (gfx950): HIP kernels and the C ABI.
//
// Replaces the CUDA driver and kernels of i6_native_ops/fbw/fbw_op.cu:17-153,226-393
// (5T+6 launches, CAS log-add, a (T,E) edge buffer) with four stages:
//
//   1. prepare   per sequence: stable partition of the edge list, local state ids, distinct
//                emission ids ("slots"), and three orderings of the edges -- by target state
//                (alpha), by source state (beta), by emission slot (combine).
//   2. gather    am_scores[t,b,emission] for the distinct emissions of sequence b -> compact rows.
//   3. recurse   one workgroup per (sequence, direction): the whole time loop runs inside the
//                kernel with the state vector double-buffered in LDS and the incoming edges of
//                each state in registers; one barrier per frame, no atomics, fixed summation order.
//   4. combine   per (frame, sequence): edge scores alpha+w+am+beta, per-frame normaliser,
//                per-emission sums, and the dense F-wide output row written with coalesced stores.
//
// Semantics follow the reference exactly (see include/i6fbw.h for the contract):
// alpha_0 = 0 at the start state (fbw_op.cu:296-302), beta seeded with 0 at the end state when
// t+1 == seq_len (fbw_op.cu:61-69), edge score +inf if either side is +inf (fbw_op.cu:83-86),
// sum_output = 0 for empty frames (fbw_op.cu:120-128), out = +inf where nothing contributes
// (fbw_op.cu:41-44,131-134,152,366-369).
//
// Parts of this translation unit: this file (kernels of the four stages, the host side of
// i6fbw_run, status, dumps), generic_path.inc (sequences beyond the capacity of those kernels),
// viterbi_kernels.inc (best path on the same tables, i6fbw_viterbi), fsa_builders.inc (CTC / HMM
// automaton arrays built on the device).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <mutex>
#include <type_traits>
#include <string>
#include <vector>

#include "../../include/i6fbw.h"

namespace {

constexpr int KMAX = 8;               // in-/out-degree held in registers by the recursion
constexpr int KWIDE = 15;             // largest degree the edge tables hold (re-read from memory per frame beyond KMAX);
                                      // the best-path search packs the edge's rank into four bits, with 15 | 4095 << 0 reserved
constexpr int EB_MAX = 8192;          // edges of one sequence (capacity of the LDS sort)
constexpr int F_BITMAP_MAX = 131072;  // emission ids covered by the LDS presence bitmap
constexpr int S_MAX = 4096;           // states of one sequence
constexpr int D_MAX = 4096;           // distinct emissions of one sequence
// states of a sequence whose two state vectors fit, as doubles, the state area of the recursion
// instance that keeps float vectors of S_MAX states (fbw_recurse_dense)
constexpr int DENSE_F64_STATES = (((S_MAX + 16) / 2 - 16) / 16) * 16;
#ifndef I6_TG
#define I6_TG 8
#endif
constexpr int TG = I6_TG;             // frames per gather workgroup
#ifndef I6_TC
#define I6_TC 8
#endif
constexpr int TC = I6_TC;             // frames per combine workgroup
#ifndef I6_FLAT_TCF
#define I6_FLAT_TCF 2
#endif
constexpr int FLAT_TCF = I6_FLAT_TCF; // frames per posterior job of the flat dense write (one flag each)
static_assert(TC % FLAT_TCF == 0, "posterior jobs tile a strip");
constexpr int RENORM = 8;             // frames between renormalisations of the state vector
constexpr int COMB_THREADS = 256;
constexpr int COMB_JD = D_MAX / COMB_THREADS;
constexpr int COMB_XS = 1024;         // edge scores staged in LDS per pass of the combine kernel
constexpr int COMB_BATCH = 4;         // frames the row writer takes together for sequences of up to COMB_BATCH_EDGES edges (rows of up to COMB_BATCH_F floats)
constexpr int COMB_BATCH_EDGES = 512, COMB_BATCH_F = 1024;
constexpr int COMB_MID_EDGES = 4096;  // up to here a combine workgroup keeps the edges of its sequence in registers ...
constexpr int COMB_MID_SLOTS = 2048;  // ... and the distinct emissions of the sequence spread over its threads' registers
#ifndef I6_FLOAT_FRAMES
#define I6_FLOAT_FRAMES 256           // sequences with more frames keep their state vectors in double (with one or two states per thread double
                                      // costs these instances nothing measurable; 177 states over 400 frames in float: 7.1e-5, in double 9.8e-6)
#endif
constexpr int REC_THREADS = 512;      // compute threads of a recursion workgroup
constexpr int REC_LOADERS = 1;        // loader waves beside them
constexpr int REC_BLOCK = REC_THREADS + 64 * REC_LOADERS;
// Two recursion workgroups share a compute unit only if a workgroup has at most eight waves
// (measured: nine-wave workgroups with this much LDS are placed one per unit): the instance for
// batches with more workgroups than compute units runs 448 compute threads beside the loader wave.
constexpr int REC_THREADS_DENSE = 448;
constexpr int REC_BLOCK_DENSE = REC_THREADS_DENSE + 64 * REC_LOADERS;
// Batches of large automata (more than BIG_STATES states per sequence on average) run the instance with
// fifteen compute waves: up to 960 states at one per thread, and half as many rounds beyond -- four
// waves per SIMD with two states each overlap their LDS and arithmetic phases better than two with four
// (8 sequences of 1350-1600 states over 2300-3700 frames: 2.83 -> 2.35 ms per call).  Small automata are
// better off with fewer waves at the barrier (headline, 350-450 states: 0.507 ms against 0.533).
constexpr int REC_THREADS_BIG = 960;
constexpr int REC_BLOCK_BIG = REC_THREADS_BIG + 64 * REC_LOADERS;
#ifndef I6_BIG_STATES
#define I6_BIG_STATES 512
#endif
constexpr int BIG_STATES = I6_BIG_STATES;
static_assert(REC_BLOCK_BIG <= 1024, "one workgroup");
constexpr unsigned NO_STATE = 0xFFFFu;
constexpr int SEQ_GENERIC = 1;        // value of SeqMeta::err / errA / errB that routes a sequence to the general path
constexpr int SCAN_BLOCK = 1024;      // edges per workgroup of the sortedness scan
constexpr int SYNC_HDR = 16;          // ints before the progress counters in the hand-off area:
                                      // [0] abort flag, [1] recursion workgroups placed so far, [3] preparation workgroups finished,
                                      // [4..5] status report {code, sequence}, [6] longest sequence of the batch in frames
constexpr int PUBLISH = 32;           // recursion steps between progress publications
constexpr int SPIN_LIMIT = 1 << 20;   // polls before a waiting wave gives up (see g_spin_limit)
// Scores are kept in units of log 2 inside the workspace (exp2/log2 are single instructions).
constexpr float LOG2E = 1.44269504088896341f;
constexpr float LN2 = 0.693147180559945309f;
#define INF_F __builtin_inff()

struct SeqMeta {
    int edge_begin;   // edges with a smaller sequence index
    int n_edges;
    int state_min;
    int S, SP;        // local states, padded to 16
    int D, DP;        // distinct emissions, padded to 16
    int L;            // frames that carry probability mass (0: none)
    int start_local, end_local;
    int err;          // common problems (written by the emission-order role)
    int Kin, errA;    // written by the target-order role
    int Kout, errB;   // written by the source-order role
    int pad;          // bit 0: edges contiguous in the input
};

__host__ __device__ inline long long round16(long long x) { return (x + 15) & ~15LL; }
// Workspace offsets of a sequence follow from the number of edges before it, so that no
// prefix sum over sequences (and no cross-workgroup dependency) is needed.
__host__ __device__ inline long long state_off(long long edge_begin, int b) { return round16(2 * edge_begin) + 32LL * b; }
__host__ __device__ inline long long slot_off(long long edge_begin, int b) { return round16(edge_begin) + 32LL * b; }
// Entries of a sequence's renumbering table (see local_state) and the home position of a state id in it
__host__ __device__ inline unsigned renum_capacity(int n_edges) { return 2u * (2u * (unsigned)n_edges + 16u); }
__host__ __device__ inline unsigned renum_home(int id, unsigned cap) {
    return (unsigned)(((unsigned long long)((unsigned)id * 2654435761u) * cap) >> 32);
}

struct Layout {
    size_t meta, sync, sortflag, seqbegin, eidx, ellA, ellB, crec, cbegin, demis, tband, renum, cflag, wpfx, offA, offB, alpha, beta, gtab, total;
    long long ss_total, gg_total;
    int wpfx_stride;      // ints per sequence in the emission rank table (0: F too large for it)
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

Layout make_layout(long long T, long long B, long long E, long long F = 1) {
    Layout l;
    l.wpfx_stride = F <= F_BITMAP_MAX ? (int)(((F + 31) >> 5) + 2) : 0;
    l.ss_total = round16(2 * E) + 32 * B + 16;
    l.gg_total = round16(E) + 32 * B + 16;
    size_t o = 0;
    l.meta = o;     o = align256(o + sizeof(SeqMeta) * B);
    l.sync = o;     o = align256(o + sizeof(int) * (SYNC_HDR + 2 * B + B * ((T + TG - 1) / TG)));
    l.sortflag = o; o = align256(o + sizeof(int) * (E / SCAN_BLOCK + 2));
    l.seqbegin = o; o = align256(o + sizeof(int) * (B + 2));
    l.eidx = o;     o = align256(o + sizeof(int) * (E + 1));
    l.ellA = o;     o = align256(o + sizeof(uint2) * KMAX * l.ss_total);
    l.ellB = o;     o = align256(o + sizeof(uint2) * KMAX * l.ss_total);
    l.crec = o;     o = align256(o + sizeof(uint4) * (E + 1));
    l.cbegin = o;   o = align256(o + sizeof(int) * l.gg_total);
    l.demis = o;    o = align256(o + sizeof(int) * l.gg_total);
    l.tband = o;    o = align256(o + sizeof(int2) * l.gg_total);
    l.renum = o;    o = align256(o + sizeof(int2) * 2 * l.ss_total);
    l.offA = o;     o = align256(o + sizeof(double) * B * T);
    l.offB = o;     o = align256(o + sizeof(double) * B * T);
    l.alpha = o;    o = align256(o + sizeof(float) * l.ss_total * T);
    l.beta = o;     o = align256(o + sizeof(float) * l.ss_total * T);
    l.gtab = o;     o = align256(o + sizeof(float) * l.gg_total * T);
    // (behind everything else: the offsets above do not depend on F)
    l.cflag = o;    o = align256(o + sizeof(int) * B * ((T + FLAT_TCF - 1) / FLAT_TCF));
    l.wpfx = o;     o = align256(o + sizeof(int) * B * l.wpfx_stride);
    l.total = o;
    return l;
}

#ifdef I6_TRACE
__device__ unsigned long long g_trace[4096];   // debug builds only: in-kernel timestamps
__device__ inline unsigned long long trace_cu_key() {
    const unsigned hw = __builtin_amdgcn_s_getreg(4 | (31 << 11)), xcc = __builtin_amdgcn_s_getreg(20 | (31 << 11));
    return ((unsigned long long)(xcc & 15u) << 32) | ((hw >> 8) & 0xffu) | 0x100000000000ull;
}
__device__ inline void trace_corun(int slot) {
    if (threadIdx.x == 0) {
        const unsigned long long k = trace_cu_key();
        int hit = 0, pair = 0;
        for (int i = 0; i < 64; i++) { const unsigned long long r = g_trace[3000 + i]; hit |= r == k; pair |= (r ^ k) == 1; }
        atomicAdd(&g_trace[slot], 1ull); if (hit) atomicAdd(&g_trace[slot + 1], 1ull); if (pair) atomicAdd(&g_trace[slot + 2], 1ull);
    }
}
#endif

// ---------------------------------------------------------------------------------------------
// small device helpers
// ---------------------------------------------------------------------------------------------
// negative: a reported problem; SEQ_GENERIC: handled by the general path; 0: fast path
__device__ inline int seq_error(const SeqMeta& m) {
    if (m.err < 0) return m.err;
    if (m.errA < 0) return m.errA;
    if (m.errB < 0) return m.errB;
    return (m.err | m.errA | m.errB) ? 1 : 0;
}

// Recursion class of a sequence: 0 nothing to do, 1..3 by size, -1 error, -2 general path.
__device__ inline int rec_class(const SeqMeta& m, const int threads = REC_THREADS) {
    const int err = seq_error(m);
    if (err < 0) return -1;
    if (m.L == 0 || m.n_edges == 0) return 0;
    if (err > 0) return -2;            // general path
    if (m.SP <= threads && m.DP <= (threads > 512 ? 1024 : 512)) return 1;     // (the loader wave of the large instance takes rows of 1024)
    if (m.SP <= 4 * threads && m.DP <= 2048) return 2;
    return 3;
}

// Hand-off between kernels that run at the same time (gather -> recursion -> combine).  The
// L2 caches of the eight XCDs are not coherent with each other inside a kernel, so everything
// that crosses kernels goes through agent-scope accesses (sc1: written through / read from the
// memory side), and a flag or counter is published only after the data stores have completed.
// Every wait is bounded: after SPIN_LIMIT polls the waiter sets the abort flag and goes on, and
// the call reports I6FBW_ERR_TIMEOUT.
__device__ __forceinline__ void store_agent(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_agent(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_agent(double* p, double v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float load_agent(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int load_agent(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ double load_agent(const double* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ unsigned long long load_agent(const unsigned long long* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool SYNC, typename T> __device__ __forceinline__ void store_x(T* p, T v) { if (SYNC) store_agent(p, v); else *p = v; }
template <bool SYNC, typename T> __device__ __forceinline__ T load_x(const T* p) { return SYNC ? load_agent(p) : *p; }
// waits until this wave's global stores have been acknowledged
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// The poll limit is a device variable so that a test can force the give-up path from the host
// (i6fbw_set_spin_limit) with every kernel still running to its normal end.
__device__ int g_spin_limit = SPIN_LIMIT;

// polls *p until it is >= want; false if it gave up (or somebody else already had to)
// (quiet: running out of polls is not an error yet, the caller tries again)
__device__ __forceinline__ bool spin_until_ge(const int* p, int want, int* abort_flag, bool quiet = false) {
    const int limit = g_spin_limit;
    for (int n = 0; n < limit; n++) {
        if (load_agent(p) >= want) return true;
        if ((n & 255) == 255 && load_agent(abort_flag)) return false;
        __builtin_amdgcn_s_sleep(2);
    }
    if (!quiet) atomicOr(abort_flag, 1);
    return false;
}

// Gather and combine workgroups are handed out (1-D grid, dispatched in index order) with the
// sequence index running fastest: workgroups that run together read / write neighbouring rows.
__device__ __forceinline__ void strip_index(int B, int* b, int* y) {
    *b = blockIdx.x % B;
    *y = blockIdx.x / B;
}

// wave-wide minimum in lane 63 (DPP row operations, no LDS traffic)
__device__ __forceinline__ float wave_min_dpp(float v) {
#define I6_DPP_MIN(ctrl, rmask)                                                                          \
    v = fminf(v, __uint_as_float((unsigned)__builtin_amdgcn_update_dpp((int)__float_as_uint(v), (int)__float_as_uint(v), \
                                                                       ctrl, rmask, 0xf, false)))
    I6_DPP_MIN(0x111, 0xf);   // row_shr:1
    I6_DPP_MIN(0x112, 0xf);   // row_shr:2
    I6_DPP_MIN(0x114, 0xf);   // row_shr:4
    I6_DPP_MIN(0x118, 0xf);   // row_shr:8  -> lane 15 of each row holds the row minimum
    I6_DPP_MIN(0x142, 0xa);   // row_bcast:15 into rows 1 and 3
    I6_DPP_MIN(0x143, 0xc);   // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave minimum
#undef I6_DPP_MIN
    return v;
}
// wave-wide sum in lane 63, fixed association order
__device__ __forceinline__ float wave_sum_dpp(float v) {
#define I6_DPP_ADD(ctrl, rmask)                                                                 \
    v += __uint_as_float((unsigned)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), ctrl, rmask, 0xf, false))
    I6_DPP_ADD(0x111, 0xf);
    I6_DPP_ADD(0x112, 0xf);
    I6_DPP_ADD(0x114, 0xf);
    I6_DPP_ADD(0x118, 0xf);
    I6_DPP_ADD(0x142, 0xa);
    I6_DPP_ADD(0x143, 0xc);
#undef I6_DPP_ADD
    return v;
}
__device__ __forceinline__ float lane63(float v) {
    return __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)__float_as_uint(v), 63));
}

// ---------------------------------------------------------------------------------------------
// stage 1: prepare
// ---------------------------------------------------------------------------------------------
struct PrepArgs {
    const int32_t* edges; long long edge_stride;
    const float* weights;
    const int32_t* start_end; long long se_stride;
    const int32_t* seq_lens;
    int T, B, F, E, n_states;
    int gate_need;      // > 0: a workgroup only ends when this many recursion workgroups are on the machine (see fbw_gate)
    int count_wgs;      // overlapped schedule: a kernel that runs beside this one waits for the count of its finished workgroups
    int best_path;      // tables for the best-path search: weights unscaled, no source-ordered table
    int no_band;        // every (frame, slot) pair is gathered (debug dumps of the forward scores)
    int force_generic;  // F is too large for the emission bitmap: every sequence takes the general path
    int dense;          // the recursion runs on the instance with the small state area (fbw_recurse_dense)
    int2* renum;        // renumbering tables, two entries per state of room (see local_state)
    SeqMeta* meta; int* sync; int* sortflag; int* seqbegin; int* eidx; uint2* ellA; uint2* ellB; uint4* crec; int* cbegin; int* demis; int2* tband;
    int* cflag = nullptr;   // per (sequence, strip of TC frames): compact posteriors written (flat dense write); may be null
    int* wpfx = nullptr;    // per sequence: number of distinct emissions below 32 * w, for w = 0 .. ceil(F / 32); may be null
    int wpfx_stride = 0;
};

// sortflag[blk] = 1 if the sequence indices of edges [blk*SCAN_BLOCK, (blk+1)*SCAN_BLOCK] never
// decrease.  Where the index steps up, the first edge of every sequence in between is recorded:
// seqbegin[q] = first edge with sequence index >= q (valid if the whole list turns out sorted).
// As the first kernel of a call it also clears the header of the hand-off area.
__global__ __launch_bounds__(256) void fbw_scan_sorted(const int32_t* e_seq, int E, int B, int* sortflag, int* seqbegin, int* sync) {
    __shared__ int bad;
    if (blockIdx.x == 0 && threadIdx.x < SYNC_HDR) sync[threadIdx.x] = 0;
    if (threadIdx.x == 0) bad = 0;
    __syncthreads();
    const int base = blockIdx.x * SCAN_BLOCK;
    int mybad = 0;
    for (int i = base + threadIdx.x; i < min(E, base + SCAN_BLOCK); i += 256) {
        const unsigned cur = (unsigned)e_seq[i];
        const unsigned prev = i > 0 ? (unsigned)e_seq[i - 1] : 0u;
        mybad |= cur < prev;
        // sequences prev+1 .. cur (from 0 for the first edge) start at edge i
        // (sequence index -1 marks a padding edge; such edges sort behind all others)
        unsigned q0 = i > 0 ? prev + 1u : 0u;
        if (!(i > 0 && prev == 0xffffffffu))
            for (unsigned q = q0; q <= min(cur, (unsigned)B); q++) seqbegin[q] = i;
        if (i == E - 1)
            for (unsigned q = min(cur, (unsigned)B) + 1u; q <= (unsigned)B; q++) seqbegin[q] = E;
    }
    if (mybad) atomicOr(&bad, 1);
    __syncthreads();
    if (threadIdx.x == 0) sortflag[blockIdx.x] = !bad;
}

__device__ inline int block_excl_scan(int v, int* wsum, int nwaves, int* total) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        int t = __shfl_up(incl, o);
        if (lane >= o) incl += t;
    }
    if (lane == 63) wsum[w] = incl;
    __syncthreads();
    int base = 0, tot = 0;
    for (int i = 0; i < nwaves; i++) {
        int x = wsum[i];
        if (i < w) base += x;
        tot += x;
    }
    __syncthreads();
    *total = tot;
    return base + incl - v;
}

// In-place bitonic sort of N (a power of two) keys in LDS by the whole workgroup.
template <int NT>
__device__ inline void lds_bitonic_sort(unsigned* keys, const int N) {
    for (int k = 2; k <= N; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < N; i += NT) {
                const int ixj = i ^ j;
                if (ixj > i) {
                    const unsigned x = keys[i], y = keys[ixj];
                    if ((x > y) == ((i & k) == 0)) { keys[i] = y; keys[ixj] = x; }
                }
            }
            __syncthreads();
        }
    }
}

// The same sort for N = R * NT keys with the keys in registers: thread tid holds the elements tid + r * NT.  Partners
// NT or more apart sit in the same thread, partners less than a wave apart are reached with a lane exchange; only the
// steps in between go through LDS (two barriers each): 18 of the 78 steps for 4096 keys on 1024 threads, where the
// loop above has a barrier behind every step.  The caller has written the keys and passed a barrier; the sorted keys
// are back in LDS behind the last barrier of this function.
template <int NT, int R>
__device__ __forceinline__ void bitonic_sort_in_registers(unsigned* keys, const int tid) {
    unsigned x[R];
#pragma unroll
    for (int r = 0; r < R; r++) x[r] = keys[tid + r * NT];
    // a step with partners j < NT apart, for the stage of run length k
    auto across_threads = [&](const int k, const int j) {
        unsigned y[R];
        if (j >= 64) {
            __syncthreads();        // the reads of the step before (the initial ones on the first)
#pragma unroll
            for (int r = 0; r < R; r++) keys[tid + r * NT] = x[r];
            __syncthreads();
#pragma unroll
            for (int r = 0; r < R; r++) y[r] = keys[(tid ^ j) + r * NT];
        } else {
#pragma unroll
            for (int r = 0; r < R; r++) y[r] = (unsigned)__shfl_xor((int)x[r], j);
        }
        const bool lower = (tid & j) == 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const bool up = ((tid + r * NT) & k) == 0;
            x[r] = (lower == up) ? min(x[r], y[r]) : max(x[r], y[r]);
        }
    };
    for (int k = 2; k <= NT; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) across_threads(k, j);
#pragma unroll
    for (int kr = 2; kr <= R; kr <<= 1) {          // stages of run length kr * NT
#pragma unroll
        for (int jr = kr >> 1; jr > 0; jr >>= 1) {
#pragma unroll
            for (int r = 0; r < R; r++)
                if ((r & jr) == 0) {
                    const bool up = (r & kr) == 0;
                    const unsigned lo = min(x[r], x[r | jr]), hi = max(x[r], x[r | jr]);
                    x[r] = up ? lo : hi;
                    x[r | jr] = up ? hi : lo;
                }
        }
        for (int j = NT >> 1; j > 0; j >>= 1) across_threads(kr * NT, j);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; r++) keys[tid + r * NT] = x[r];
    __syncthreads();
}

constexpr int PREP_AUX_WORDS = 2048;   // scratch words of a preparation workgroup beside its sort keys
constexpr int KEY_POS_BITS = 13;   // EB_MAX = 2^13 positions; the primary key sits above them
static_assert((1 << KEY_POS_BITS) == EB_MAX, "key layout");

// first index i in [0,n) with (keys[i] >> KEY_POS_BITS) >= p
__device__ inline int lower_bound_hi(const unsigned* keys, int n, unsigned p) {
    int lo = 0, hi = n;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if ((keys[mid] >> KEY_POS_BITS) < p) lo = mid + 1; else hi = mid;
    }
    return lo;
}
// Lower bound on the number of edges of any path from state id `from` to state id `to` when no
// edge raises the id by more than dmax or lowers it by more than -dmin.  Exact for left-to-right
// chains numbered along the chain; never larger than the true distance for any automaton.
__device__ inline int min_steps(int from, int to, int dmax, int dmin) {
    const int diff = to - from;
    if (diff == 0) return 0;
    if (diff > 0) return dmax > 0 ? (diff + dmax - 1) / dmax : (1 << 30);
    return dmin < 0 ? (-diff - dmin - 1) / -dmin : (1 << 30);
}

// grid (3, B): role 0 orders the edges of sequence b by target state (alpha), role 1 by source
// state (beta), role 2 by emission slot (combine) and writes the shared part of the meta record.
// For edge lists grouped by sequence (the usual case) the scan kernel has recorded where each
// sequence starts; any other order is handled by a stable scan over the whole list.
template <int NT>
__device__ __forceinline__ void prepare_sequence(const PrepArgs& a, unsigned* lds) {
    // dynamic LDS: sort keys, a scratch area (see by_level), then the emission bitmap and its prefix counts (one word per 32 classes)
    unsigned* keys = lds;
    unsigned* aux = lds + EB_MAX;
    unsigned* bitmap = aux + PREP_AUX_WORDS;
    int* wordpfx = (int*)(bitmap + ((a.F + 31) >> 5));
    __shared__ int wsum[NT / 64];
    __shared__ int s_lt, s_bad, s_kmax, s_sorted, s_dmax, s_dmin, s_count, s_nonmono;
    __shared__ unsigned s_min, s_max;

    const int role = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    // what depends on nothing but the sequence index is requested before anything is waited for (seq_first / seq_next: where
    // the edges of this sequence and of the next one begin if the list is grouped by sequence, see fbw_scan_sorted)
    const int seq_first = a.E > 0 ? a.seqbegin[b] : 0, seq_next = a.E > 0 ? a.seqbegin[b + 1] : 0;
    const unsigned st_state = (unsigned)a.start_end[b], en_state = (unsigned)a.start_end[a.se_stride + b];
    const unsigned sl = (unsigned)a.seq_lens[b];
    const int32_t* e_from = a.edges;
    const int32_t* e_to = a.edges + a.edge_stride;
    const int32_t* e_emis = a.edges + 2 * a.edge_stride;
    const int32_t* e_seq = a.edges + 3 * a.edge_stride;
    const int E = a.E;

    if (tid == 0) { s_lt = 0; s_bad = 0; s_kmax = 0; s_sorted = 1; s_min = 0xffffffffu; s_max = 0u; s_dmax = 0; s_dmin = 0; s_count = 0; s_nonmono = 0; }
    __syncthreads();
    const int nflag = (E + SCAN_BLOCK - 1) / SCAN_BLOCK;
    int unsorted = 0;
    for (int i = tid; i < nflag; i += NT) unsorted |= !a.sortflag[i];
    if (unsorted) atomicAnd(&s_sorted, 0);
    __syncthreads();
    const bool sorted = s_sorted != 0;

    int edge_begin, n_edges, pos = 0;
    int bad = 0, nonmono = 0;         // nonmono: some edge leads to a state with a smaller id
    unsigned mn = 0xffffffffu, mx = 0u;
    const int chunk = (E + NT - 1) / NT;
    const int lo = min(E, tid * chunk), hi = min(E, lo + chunk);
    if (sorted) {
        edge_begin = seq_first;
        n_edges = seq_next - seq_first;
        if (b == 0 && E > 0 && (unsigned)e_seq[E - 1] >= (unsigned)a.B && (unsigned)e_seq[E - 1] != 0xffffffffu) bad = 1;
        for (int i = edge_begin + tid; i < edge_begin + n_edges; i += NT) {
            unsigned f = (unsigned)e_from[i], t = (unsigned)e_to[i];
            mn = min(mn, min(f, t)); mx = max(mx, max(f, t));
            nonmono |= t < f;
            if (f >= (unsigned)a.n_states || t >= (unsigned)a.n_states || (unsigned)e_emis[i] >= (unsigned)a.F) bad = 1;
        }
        if (bad) atomicOr(&s_bad, 1);
        if (nonmono) atomicOr(&s_nonmono, 1);
        if (mn <= mx) { atomicMin(&s_min, mn); atomicMax(&s_max, mx); }
        __syncthreads();
    } else {
        // count the edges of earlier sequences and of this one, state range, index checks
        int lt = 0, eq = 0;
        for (int i = lo; i < hi; i++) {
            unsigned s = (unsigned)e_seq[i];
            lt += s < (unsigned)b;
            if (s == (unsigned)b) {
                eq++;
                unsigned f = (unsigned)e_from[i], t = (unsigned)e_to[i];
                mn = min(mn, min(f, t)); mx = max(mx, max(f, t));
                nonmono |= t < f;
                if (f >= (unsigned)a.n_states || t >= (unsigned)a.n_states || (unsigned)e_emis[i] >= (unsigned)a.F) bad = 1;
            }
            if (b == 0 && s >= (unsigned)a.B && s != 0xffffffffu) bad = 1;
        }
        if (lt) atomicAdd(&s_lt, lt);
        if (bad) atomicOr(&s_bad, 1);
        if (nonmono) atomicOr(&s_nonmono, 1);
        if (eq) { atomicMin(&s_min, mn); atomicMax(&s_max, mx); }
        pos = block_excl_scan(eq, wsum, NT / 64, &n_edges);   // barriers inside publish the atomics too
        edge_begin = s_lt;
    }

    unsigned smin = min(min(s_min, st_state), en_state), smax = max(max(s_max, st_state), en_state);
    int err = 0;
    if (s_bad || st_state >= (unsigned)a.n_states || en_state >= (unsigned)a.n_states) err = I6FBW_ERR_BAD_INDEX;
    // Sequences beyond the capacity of the fast kernels take the general path (generic_path.inc,
    // generic_viterbi).
    int generic = 0;
    if (!err && n_edges > EB_MAX) generic = 1;
    // full sum: a length outside [1, T] leaves the sequence without probability mass; best path:
    // lengths beyond T are read as T
    const int L = a.best_path ? ((int)sl < 0 ? 0 : min((int)sl, a.T)) : ((sl >= 1u && sl <= (unsigned)a.T) ? (int)sl : 0);
    long long S = (long long)smax - smin + 1;
    // ids spread over a range much larger than their number (the workspace is sized by the edge
    // count): the states get dense numbers (below), and the sequence takes the general path, which
    // looks them up
    const bool sparse = !err && n_edges > 0 && S > 2LL * n_edges + 2;
    // up to this many edges the renumbering is done in LDS, the same way by all three roles, and the
    // sequence stays on the fast kernels: the 2n+2 ids fit the key array, and afterwards the n edge
    // keys its lower half and the distinct ids its upper half
    constexpr int RENUM_LDS_EDGES = EB_MAX / 2 - 1;
    // Sequences whose ids, spread or not, do not follow the automaton (some edge leads to a smaller id) get numbers along
    // the automaton where that matters (by_level below): that is what the recursion's renormalisation over live states
    // and the activity band of the gather go by (live_window, min_steps).
    const bool unordered = !err && n_edges > 0 && s_nonmono != 0 && s_bad == 0 && n_edges <= RENUM_LDS_EDGES && !a.force_generic;
    // ... and such a sequence is ranked too when its ids, without being spread by the measure above, span more than the
    // numbering below can hold, as the ids of one sequence among many do after a permutation over the whole batch (a chain
    // of 1020 states with ids out of 3573, 1100 frames: 7.9e-5 before): the span says nothing about the number of states then
    constexpr int LEVEL_STATES = EB_MAX / 4;
    const bool span_too_wide = unordered && !sparse && S > LEVEL_STATES && L > 0 && 5LL * S > 4LL * L;
    bool ranked = (sparse || span_too_wide) && n_edges <= RENUM_LDS_EDGES && !a.force_generic;
    if (sparse && !ranked) generic = 1;
    if (n_edges == 0) S = 1;
    if (!err && !sparse && !ranked && S > S_MAX) generic = 1;
    if (!err && a.force_generic && n_edges > 0) generic = 1;
    const long long soff = state_off(edge_begin, b), goff = slot_off(edge_begin, b);

    // i-th edge of this sequence in input order
    int* eidx = a.eidx + edge_begin;
    auto edge_at = [&](int i) -> int { return sorted ? edge_begin + i : eidx[i]; };

    int D = 0;
    if (!err && n_edges > 0 && !sorted) {
        // stable list of this sequence's edge indices (every role writes the same values)
        for (int i = lo; i < hi; i++)
            if ((unsigned)e_seq[i] == (unsigned)b) eidx[pos++] = i;
    }
    // Widely spread ids, in LDS: all ids the sequence names are sorted, the distinct ones are kept in
    // ascending order in the upper half of the key array, and a state's number is its rank there
    // (binary search).  Every role arrives at the same numbers.
    unsigned* uniq = keys + EB_MAX / 2;
    if (ranked) {
        __syncthreads();        // the edge list written above
        const int M = 2 * n_edges + 2;
        int N2 = 2;
        while (N2 < M) N2 <<= 1;
        for (int i = tid; i < N2; i += NT) {
            unsigned k = ~0u;
            if (i < 2 * n_edges) { const int e = edge_at(i >> 1); k = (unsigned)((i & 1) ? e_to[e] : e_from[e]); }
            else if (i == 2 * n_edges) k = st_state;
            else if (i == 2 * n_edges + 1) k = en_state;
            keys[i] = k;
        }
        __syncthreads();
        lds_bitonic_sort<NT>(keys, N2);
        constexpr int CH = EB_MAX / NT;
        unsigned mine[CH];
        int cnt = 0;
#pragma unroll
        for (int j = 0; j < CH; j++) {
            const int i = tid * CH + j;
            mine[j] = ~0u;
            if (i < M && (i == 0 || keys[i - 1] != keys[i])) { mine[j] = keys[i]; cnt++; }
        }
        int total;
        int at = block_excl_scan(cnt, wsum, NT / 64, &total);       // its barriers come after every read above
        S = total;
        if (total > S_MAX) { ranked = false; generic = 1; }          // too many states for the fast kernels (and for the upper half)
        else {
#pragma unroll
            for (int j = 0; j < CH; j++)
                if (mine[j] != ~0u) uniq[at++] = mine[j];
        }
        __syncthreads();
    }
    // The recursion instance for batches of more sequences than half the compute units has room for
    // double-precision state vectors of DENSE_F64_STATES states only: a larger sequence that needs them
    // (recurse_workgroup) takes the general path, which keeps its vectors in double in memory.
    if (!err && a.dense && !a.best_path && S > DENSE_F64_STATES && (5LL * S > 3LL * L || L > I6_FLOAT_FRAMES)) generic = 1;
    // rank of a state id among the distinct ids of the sequence (ids that are not spread: place in their range)
    auto rank_of = [&](const unsigned id) -> unsigned {
        if (!ranked) return id - smin;
        int lo_ = 0, hi_ = (int)S;
        while (lo_ < hi_) {
            const int mid = (lo_ + hi_) >> 1;
            if (uniq[mid] < id) lo_ = mid + 1; else hi_ = mid;
        }
        return (unsigned)lo_;
    };
    // Numbers along the automaton for a sequence whose ids do not follow it, where that matters: a tightly aligned one,
    // fewer than five frames for every four states (chains of 1021 states over 1021-1100 frames came out at 9.9e-5 under
    // permuted ids; the long-form configuration, whose optional states carry the highest ids, is at 2.5e-5 with 1.6
    // frames per state and would pay 0.17 ms per call).  A state's height is the length of the longest path from it,
    // self-loops aside, so every other edge leads to a lower state, and the states are numbered by falling height, then
    // by id.  Heights by policy iteration: every state picks the highest of its successors, the heights along the chosen
    // chains are added up by pointer jumping (log2 S rounds), and the states pick again, until every state sits exactly
    // one above its highest successor -- two or three picks for a chain with optional states, whatever the order of
    // ids and edges (one round per state, as relaxation needs, cost such a call a millisecond).  An automaton that has
    // not come to rest after LEVEL_PICKS picks (a cycle through several states never does) keeps the ranks of its ids, as
    // does one with more than LEVEL_STATES states.  Every role arrives at the same numbers.
    constexpr int LEVEL_PICKS = 8;
    static_assert(LEVEL_STATES <= PREP_AUX_WORDS && LEVEL_STATES <= 4096, "height << 16 | state; sort key height << 12 | state");
    unsigned* dn = uniq + LEVEL_STATES;          // [S]: hops to the end of the chain of chosen successors << 16 | that end; later: the state's number
    bool by_level = unordered && (ranked || !sparse) && !generic && S <= LEVEL_STATES && L > 0 && 5LL * S > 4LL * L;
    if (by_level) {
        unsigned* pk = keys;                      // the edges as ranks: source | target << 16
        unsigned* cand = aux;                     // [S]: (height of the best successor + 1) << 16 | that successor
        constexpr int SPT = LEVEL_STATES / NT;    // states per thread
        const int nS = (int)S;
        __syncthreads();        // the edge list written above (an edge list that is not grouped by sequence is read through it)
        for (int i = tid; i < n_edges; i += NT) {
            const int e = edge_at(i);
            pk[i] = rank_of((unsigned)e_from[e]) | (rank_of((unsigned)e_to[e]) << 16);
        }
        for (int r = tid; r < nS; r += NT) dn[r] = (unsigned)r;
        __syncthreads();
        bool rest = false;
        for (int pick = 0; pick < LEVEL_PICKS && !rest; pick++) {
            for (int r = tid; r < nS; r += NT) cand[r] = 0u;
            __syncthreads();
            for (int i = tid; i < n_edges; i += NT) {
                const unsigned u = pk[i] & 0xFFFFu, w = pk[i] >> 16;
                if (u != w) atomicMax(&cand[u], (((dn[w] >> 16) + 1u) << 16) | w);
            }
            __syncthreads();
            int off = 0;
            for (int r = tid; r < nS; r += NT) off |= (cand[r] >> 16) != (dn[r] >> 16);
            if (!__syncthreads_or(off)) { rest = true; break; }
            for (int r = tid; r < nS; r += NT) { const unsigned c = cand[r]; dn[r] = c ? (1u << 16) | (c & 0xFFFFu) : (unsigned)r; }
            __syncthreads();
            for (int span = 1; span < nS; span <<= 1) {
                unsigned q[SPT];
#pragma unroll
                for (int j = 0; j < SPT; j++) {
                    const int r = tid + j * NT;
                    q[j] = 0u;
                    if (r < nS) {
                        const unsigned a_ = dn[r], b_ = dn[a_ & 0xFFFFu];
                        q[j] = (min((a_ >> 16) + (b_ >> 16), 4095u) << 16) | (b_ & 0xFFFFu);      // (a cycle saturates and never comes to rest)
                    }
                }
                __syncthreads();
#pragma unroll
                for (int j = 0; j < SPT; j++)
                    if (tid + j * NT < nS) dn[tid + j * NT] = q[j];
                __syncthreads();
            }
        }
        if (!rest) by_level = false;
        else {
            int N3 = 2;
            while (N3 < nS) N3 <<= 1;
            for (int i = tid; i < N3; i += NT) keys[i] = i < nS ? ((4095u - (dn[i] >> 16)) << 12) | (unsigned)i : ~0u;
            __syncthreads();
            lds_bitonic_sort<NT>(keys, N3);
            for (int i = tid; i < nS; i += NT) dn[keys[i] & 0xFFFu] = (unsigned)i;
            __syncthreads();
        }
    }
    // state id -> number within the sequence
    auto local = [&](const unsigned id) -> unsigned {
        const unsigned r = rank_of(id);
        return by_level ? dn[r] : r;
    };
    int SP = (int)round16(S);
    if (!err && !generic && n_edges > 0) {
        // emission presence bitmap -> slot = rank of the emission id among the distinct ones
        const int nwords = (a.F + 31) >> 5;
        for (int w = tid; w < nwords; w += NT) bitmap[w] = 0u;
        __syncthreads();
        for (int i = tid; i < n_edges; i += NT) {
            unsigned em = (unsigned)e_emis[edge_at(i)];
            atomicOr(&bitmap[em >> 5], 1u << (em & 31));
        }
        __syncthreads();
        const int wpt = (nwords + NT - 1) / NT;
        const int w0 = min(nwords, tid * wpt), w1 = min(nwords, w0 + wpt);
        int c = 0;
        for (int w = w0; w < w1; w++) c += __popc(bitmap[w]);
        int run = block_excl_scan(c, wsum, NT / 64, &D);
        for (int w = w0; w < w1; w++) { wordpfx[w] = run; run += __popc(bitmap[w]); }
        __syncthreads();
        if (D > D_MAX) generic = 1;
        if (role == 2 && a.wpfx) {
            // the rank table also goes to memory: the flat dense write finds with it the slots whose
            // emission falls into a piece of a row
            int* wp = a.wpfx + (size_t)b * a.wpfx_stride;
            for (int w = tid; w < nwords + 2; w += NT) wp[w] = w < nwords ? wordpfx[w] : D;
        }
    }
    const int DP = (int)round16(D > 0 ? D : 1);

    int start_loc = (int)local(st_state), end_loc = (int)local(en_state);
    if ((sparse || ranked || by_level) && role == 2) {
        // The general path looks the numbers up in an open-addressing table {id + 1, number} (see
        // local_state), which is written for every sequence whose numbers are not simply the place of the
        // id in its range: the other two roles may still send it there.  Numbers: the ones from above,
        // or, for a sequence with spread ids that is too large for that, the order in which the ids happen
        // to be entered (any numbering will do: the general path never compares ids, and the distance
        // bounds of min_steps hold for every numbering).
        const bool numbered = ranked || !sparse;
        int2* tab = a.renum + 2 * soff;
        const unsigned cap = renum_capacity(n_edges);
        for (unsigned i = tid; i < cap; i += NT) { store_agent(&tab[i].x, 0); store_agent(&tab[i].y, 0); }
        wait_stores();
        __syncthreads();        // also: the edge list written above
        auto enter = [&](const int id) {
            unsigned h = renum_home(id, cap);
            while (true) {
                const int seen = atomicCAS(&tab[h].x, 0, id + 1);
                if (seen == 0) { store_agent(&tab[h].y, numbered ? (int)local((unsigned)id) : atomicAdd(&s_count, 1)); return; }
                if (seen == id + 1) return;
                h = h + 1 == cap ? 0 : h + 1;
            }
        };
        auto number_of = [&](const int id) -> int {
            unsigned h = renum_home(id, cap);
            while (true) {
                const int key = load_agent(&tab[h].x);
                if (key == id + 1) return load_agent(&tab[h].y);
                if (key == 0) return 0;
                h = h + 1 == cap ? 0 : h + 1;
            }
        };
        for (int i = tid; i < n_edges; i += NT) {
            const int e = edge_at(i);
            enter(e_from[e]);
            enter(e_to[e]);
        }
        if (tid == 0) { enter((int)st_state); enter((int)en_state); }
        wait_stores();
        __syncthreads();
        if (!numbered) {
            S = s_count;
            SP = (int)round16(S);
            start_loc = number_of((int)st_state);
            end_loc = number_of((int)en_state);
        }
    }

    if (role == 2) {
        // hand-off area of this sequence: progress counters and gather flags start at zero
        const int nstrip = (a.T + TG - 1) / TG;
        if (tid < 2) a.sync[SYNC_HDR + 2 * b + tid] = 0;
        int* gf = a.sync + SYNC_HDR + 2 * a.B + (size_t)b * nstrip;
        for (int i = tid; i < nstrip; i += NT) gf[i] = 0;
        if (a.cflag) {
            const int ncf = (a.T + FLAT_TCF - 1) / FLAT_TCF;
            int* cf = a.cflag + (size_t)b * ncf;
            for (int i = tid; i < ncf; i += NT) cf[i] = 0;
        }
        if (tid == 0) atomicMax(&a.sync[6], L);      // longest sequence of the batch (header cleared by the scan kernel)
    }
    if (role == 2 && tid == 0) {
        SeqMeta* m = a.meta + b;
        m->edge_begin = edge_begin; m->n_edges = n_edges; m->state_min = (int)smin;
        m->S = (int)S; m->SP = SP; m->D = D; m->DP = DP; m->L = L;
        m->start_local = start_loc; m->end_local = end_loc;
        m->err = err ? err : (generic ? SEQ_GENERIC : 0);
        // bit 0: the edges of the sequence are contiguous in the input; bit 1: its states are renumbered;
        // bits 8 and up: see below
        m->pad = (sorted ? 1 : 0) | ((sparse || ranked || by_level) ? 2 : 0);
    }
    if (err || generic || n_edges == 0) {
        if (tid == 0) {
            if (role == 0) { a.meta[b].Kin = 0; a.meta[b].errA = 0; }
            if (role == 1) { a.meta[b].Kout = 0; a.meta[b].errB = 0; }
        }
        return;
    }

    if (a.best_path && role == 1) {
        if (tid == 0) { a.meta[b].Kout = 0; a.meta[b].errB = 0; }
        return;
    }
    const float wscale = a.best_path ? 1.f : LOG2E;

    auto slot_of = [&](unsigned em) -> unsigned {
        return (unsigned)wordpfx[em >> 5] + (unsigned)__popc(bitmap[em >> 5] & ((1u << (em & 31)) - 1u));
    };

    // sort keys: (primary << 13) | position in input order; ties keep the input order
    int N = NT;                       // at least one key per thread, see below
    while (N < n_edges) N <<= 1;
    for (int i = tid; i < N; i += NT) {
        unsigned k = ~0u;
        if (i < n_edges) {
            int e = edge_at(i);
            unsigned p = role == 0 ? local((unsigned)e_to[e]) : role == 1 ? local((unsigned)e_from[e]) : slot_of((unsigned)e_emis[e]);
            k = (p << KEY_POS_BITS) | (unsigned)i;
        }
        keys[i] = k;
    }
    __syncthreads();
    if (N == NT) {
        // one key per thread: partners less than a wave apart are reached with a lane exchange, so
        // only 10 of the 55 compare-exchange steps go through LDS and barriers
        unsigned x = keys[tid];
        for (int k = 2; k <= NT; k <<= 1) {
            for (int j = k >> 1; j > 0; j >>= 1) {
                unsigned y;
                if (j >= 64) {
                    keys[tid] = x;
                    __syncthreads();
                    y = keys[tid ^ j];
                    __syncthreads();
                } else {
                    y = (unsigned)__shfl_xor((int)x, j);
                }
                const bool up = (tid & k) == 0, lower = (tid & j) == 0;
                x = (lower == up) ? min(x, y) : max(x, y);
            }
        }
        keys[tid] = x;
        __syncthreads();
    }
    else if (N == 2 * NT) bitonic_sort_in_registers<NT, 2>(keys, tid);
    else if (N == 4 * NT) bitonic_sort_in_registers<NT, 4>(keys, tid);
    else if (N == 8 * NT) bitonic_sort_in_registers<NT, 8>(keys, tid);
    else if (EB_MAX >= 16 * NT && N == 16 * NT) bitonic_sort_in_registers<NT, (EB_MAX >= 16 * NT ? 16 : 1)>(keys, tid);
    else lds_bitonic_sort<NT>(keys, N);
    constexpr unsigned POS_MASK = (1u << KEY_POS_BITS) - 1u;

    if (role < 2) {
        // ELL table: entry (k, s) = k-th edge (in input order) entering (role 0) / leaving (role 1)
        // local state s, as {other state | slot << 16, weight * log2(e) (best path: weight)}; unused entries point at
        // NO_STATE.
        uint2* ell = (role == 0 ? a.ellA : a.ellB) + (size_t)KMAX * soff;
        int kmax = 0;
        for (int i = tid; i < n_edges; i += NT) {
            unsigned p = keys[i] >> KEY_POS_BITS;
            kmax = max(kmax, i - lower_bound_hi(keys, n_edges, p) + 1);
        }
        if (kmax) atomicMax(&s_kmax, kmax);
        __syncthreads();
        const int K = s_kmax;
        // Up to KMAX edges per state fit every sequence's share of the table area (KMAX entries per
        // state).  A larger degree, up to KWIDE, is taken as long as the table still fits the share
        // -- it does unless most states have few edges; the recursion then re-reads the table each
        // frame.  Beyond that: general path.
        const long long share = state_off((long long)edge_begin + n_edges, b + 1) - soff;
        const bool fits = K <= KMAX || (K <= KWIDE && (long long)K * SP <= (long long)KMAX * share);
        const int kerr = fits ? 0 : SEQ_GENERIC;
        if (tid == 0) {
            if (role == 0) { a.meta[b].Kin = K; a.meta[b].errA = kerr; }
            else { a.meta[b].Kout = K; a.meta[b].errB = kerr; }
        }
        if (kerr) return;
        for (int i = tid; i < K * SP; i += NT) ell[i] = make_uint2(NO_STATE, 0u);
        __syncthreads();
        for (int i = tid; i < n_edges; i += NT) {
            unsigned p = keys[i] >> KEY_POS_BITS;
            int k = i - lower_bound_hi(keys, n_edges, p);
            int e = edge_at((int)(keys[i] & POS_MASK));
            unsigned other = local(role == 0 ? (unsigned)e_from[e] : (unsigned)e_to[e]);
            unsigned slot = slot_of((unsigned)e_emis[e]);
            ell[(size_t)k * SP + p] = make_uint2(other | (slot << 16), __float_as_uint(a.weights[e] * wscale));
        }
    } else {
        // combine order: edges sorted by slot; CSR begin per slot; list of distinct emission ids
        uint4* crec = a.crec + edge_begin;
        for (int i = tid; i < n_edges; i += NT) {
            int e = edge_at((int)(keys[i] & POS_MASK));
            unsigned f = local((unsigned)e_from[e]), t = local((unsigned)e_to[e]);
            crec[i] = make_uint4(f | (t << 16), __float_as_uint(a.weights[e] * LOG2E), keys[i] >> KEY_POS_BITS, 0u);
        }
        int* cb = a.cbegin + goff;
        for (int d = tid; d <= D; d += NT) cb[d] = d == D ? n_edges : lower_bound_hi(keys, n_edges, (unsigned)d);
        int* de = a.demis + goff;
        const int nwords = (a.F + 31) >> 5;
        for (int w = tid; w < nwords; w += NT) {
            unsigned bits = bitmap[w];
            int r = wordpfx[w];
            while (bits) {
                int bit = __ffs((int)bits) - 1;
                de[r++] = w * 32 + bit;
                bits &= bits - 1;
            }
        }
        for (int d = D + tid; d < DP; d += NT) de[d] = 0;

        // Frames in which a slot can carry probability mass.  An edge u->v is dead at frame t if
        // u cannot be reached from the start state in t edges or the end state cannot be reached
        // from v in L-1-t edges; min_steps bounds both from below.  The gather writes +inf for
        // (frame, slot) pairs outside [tlo, thi] instead of reading am_scores: every edge of the
        // slot is dead there, so the result is the same, the states involved drop out of the
        // renormalisation, and for chain-like automata about half of the gather disappears.
        int dmax = 0, dmin = 0;
        for (int i = tid; i < n_edges; i += NT) {
            const int e = edge_at(i);
            const int df = (int)local((unsigned)e_to[e]) - (int)local((unsigned)e_from[e]);
            dmax = max(dmax, df); dmin = min(dmin, df);
        }
        if (dmax > 0) atomicMax(&s_dmax, dmax);
        if (dmin < 0) atomicMin(&s_dmin, dmin);
        __syncthreads();
        dmax = s_dmax; dmin = s_dmin;
        const int s_loc = start_loc, e_loc = end_loc;
        // for the recursion's renormalisation (see live_window): no edge lowers the state number, none raises it by more than dmax
        if (tid == 0 && dmin == 0 && dmax > 0 && dmax < (1 << 20) && s_loc <= e_loc) a.meta[b].pad |= dmax << 8;
        // one thread per edge; the per-slot minimum / maximum is taken with LDS atomics in the
        // memory of the sort keys (and of the distinct ids of a renumbered sequence), which is not
        // needed any more once each thread has worked out the frames of its own edges
        constexpr int EPT = EB_MAX / NT;
        int slot_[EPT], from_[EPT], upto_[EPT];     // slot of my edges (-1: none), first and last live frame
#pragma unroll
        for (int j = 0; j < EPT; j++) { slot_[j] = -1; from_[j] = 0; upto_[j] = -1; }
#pragma unroll
        for (int j = 0; j < EPT; j++) {
            // (the whole workgroup leaves at the first round without edges: a sequence of a few hundred edges has one or
            // two, and every further one cost a microsecond although no lane had anything to do in it -- 15 of the 37 us
            // of the preparation of 256 CTC automata)
            if (j * NT >= n_edges) break;
            if (tid + j * NT < n_edges) {
                const unsigned key = keys[tid + j * NT];
                const int e = edge_at((int)(key & POS_MASK));
                const int u = (int)local((unsigned)e_from[e]), v = (int)local((unsigned)e_to[e]);
                const int a1 = min_steps(v, e_loc, dmax, dmin);
                slot_[j] = (int)(key >> KEY_POS_BITS);
                from_[j] = min_steps(s_loc, u, dmax, dmin);
                upto_[j] = a1 <= L - 1 ? L - 1 - a1 : -1;
            }
        }
        __syncthreads();
        int* s_tlo = (int*)keys;
        int* s_thi = (int*)keys + D_MAX;
        static_assert(2 * D_MAX <= EB_MAX, "band arrays reuse the key array");
        for (int d = tid; d < DP; d += NT) { s_tlo[d] = d < D ? (1 << 30) : 1; s_thi[d] = d < D ? -1 : 0; }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < EPT; j++) {
            if (slot_[j] >= 0) {
                atomicMin(&s_tlo[slot_[j]], from_[j]);
                if (upto_[j] >= 0) atomicMax(&s_thi[slot_[j]], upto_[j]);
            }
        }
        __syncthreads();
        int2* tb = a.tband + goff;
        // (the best-path search reads every frame: values outside the band would have to be -inf there)
        for (int d = tid; d < DP; d += NT) tb[d] = (a.best_path || a.no_band) ? make_int2(0, 1 << 30) : make_int2(s_tlo[d], s_thi[d]);
    }
}

template <int NT>
__global__ __launch_bounds__(NT) void fbw_prepare(PrepArgs a) {
    extern __shared__ unsigned prep_lds[];
    prepare_sequence<NT>(a, prep_lds);      // every exit from it is taken by the whole workgroup

    // The recursion kernel of the overlapped schedule is already on the machine and waits for this
    // count: write this workgroup's tables back from the L2 of its XCD before it is raised.
    // (Stage after stage nobody waits for the count, and the end of the kernel does what the fence does.  The fence
    // writes the dirty lines of an L2 back, once per workgroup: the kernel's time grew by 0.09 us with every sequence
    // of the batch, whatever the workgroup size; 256 sequences: 38 -> 22 us.)
    if (!a.count_wgs) return;
    __syncthreads();
    if (threadIdx.x == 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");      // (the release half is all the writer needs: no invalidate)
        atomicAdd(&a.sync[3], 1);
        // In place of the gate kernel, where the recursion was started ahead of this kernel: the gather
        // follows in stream order, i.e. when the last of these workgroups has seen the recursion placed.
        if (a.gate_need > 0) spin_until_ge(a.sync + 1, a.gate_need, a.sync);
    }
}

// ---------------------------------------------------------------------------------------------
// stage 2: gather  gtab[b][t][slot] = log2(e) * am[t, b, demis[b][slot]]  for t < L_b.
// Strips of TG frames are handed out from both ends of a sequence towards its middle, the order in
// which the two recursions consume them.  With SYNC the rows are written through and a flag per
// strip tells the recursion (running at the same time) that the strip is complete.
// ---------------------------------------------------------------------------------------------
struct GatherArgs {
    const float* am; long long st_t, st_b;
    int T, B;
    const SeqMeta* meta; const int* demis; const int2* tband; float* gtab;
    int* sync;
    float scale;      // log2(e) for -log scores, -log2(e) for log scores
    int ascending;    // strips in ascending order (one consumer walking forward) instead of from both ends inwards
};

template <bool SYNC>
__global__ __launch_bounds__(256) void fbw_gather(GatherArgs a) {
    int b, y;
    strip_index(a.B, &b, &y);
#ifdef I6_TRACE
    trace_corun(3110);
#endif
    const SeqMeta m = a.meta[b];
    if (rec_class(m) <= 0) return;
    const int n = (m.L + TG - 1) / TG;
    if (y >= n) return;
    const int j = a.ascending ? y : ((y & 1) ? n - 1 - (y >> 1) : (y >> 1));
    const int t0 = j * TG;
    const long long goff = slot_off(m.edge_begin, b);
    const int* de = a.demis + goff;
    float* g = a.gtab + (size_t)a.T * goff;
    const float* am = a.am + (long long)b * a.st_b;
    const int nt = min(TG, m.L - t0);
    const int2* tb = a.tband + goff;
    for (int idx = threadIdx.x; idx < m.DP; idx += 256) {
        const int e = de[idx];
        const int2 band = tb[idx];        // frames outside [band.x, band.y] get +inf without a read
        float v[TG];
#pragma unroll
        for (int tt = 0; tt < TG; tt++) {
            v[tt] = INF_F;
            if (tt < nt && t0 + tt >= band.x && t0 + tt <= band.y) v[tt] = __builtin_nontemporal_load(&am[(long long)(t0 + tt) * a.st_t + e]);   // read once: keep it out of the caches
        }
#pragma unroll
        for (int tt = 0; tt < TG; tt++)
            if (tt < nt) store_x<SYNC>(&g[(size_t)(t0 + tt) * m.DP + idx], v[tt] == INF_F ? INF_F : v[tt] * a.scale);
    }
    if (SYNC) {
        wait_stores();
        __syncthreads();
        if (threadIdx.x == 0) store_agent(&a.sync[SYNC_HDR + 2 * a.B + (size_t)b * ((a.T + TG - 1) / TG) + j], 1);
    }
#ifdef I6_TRACE
    if (threadIdx.x == 0) { atomicMax(&g_trace[1], wall_clock64()); atomicMin(&g_trace[0], wall_clock64()); if (b == 0) g_trace[512 + j] = wall_clock64(); }
#endif
}

// ---------------------------------------------------------------------------------------------
// stage 3: recursion.  Workgroup 2b walks alpha of sequence b forward, workgroup 2b+1 walks beta
// backward.  Rows stored for frame t: alpha_t (state vector before frame t is consumed) and
// beta_{t+1} (after it), in units of log 2, each relative to an offset kept in double precision.
// With SYNC the loader wave waits for the gather flags, the rows are written through, and the
// number of finished rows is published every PUBLISH steps for the combine kernel.
// ---------------------------------------------------------------------------------------------
#include "generic_path.inc"

struct RecArgs {
    GenArgs gen;
    int T, B;
    int prep_wgs;     // workgroups of the preparation kernel
    const SeqMeta* meta; const uint2* ellA; const uint2* ellB; const float* gtab; float* gtab_rw;
    float* alpha; float* beta; double* offA; double* offB;
    int* sync;
};

// Barrier for LDS traffic only: waits for this wave's LDS operations and not for its global
// memory traffic (the compute waves' row stores, the loader wave's prefetches).  The memory
// clobber is what tells the compiler that other waves change the LDS buffers in between, so the
// pointers to those buffers must not be declared restrict.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Two ints behind the 32 floats of per-wave minima in a recursion workgroup's LDS: [0] whether the
// workgroup runs at all (the wait for the preparation), [1] set by the loader wave when one of
// its waits has run out.
__device__ __forceinline__ int* rec_go_flag(float* wmin) { return (int*)(wmin + 32); }
__device__ __forceinline__ int* rec_gave_up(float* wmin) { return (int*)(wmin + 32) + 1; }

struct RecCursor {
    float* wp; long long wstep;      // workspace row written by the next step
    double* op; int ostep;           // its offset
    double c; bool pending;          // running offset, renormalisation requested by the last step
    int* progress; int nsteps;       // rows finished so far (SYNC), number of steps
    const int* gave_up;              // LDS word the loader wave sets when a wait of its own has run out
    // for live_states: start and end state, largest rise of the state number along an edge (0: not known), frames,
    // direction, and the two moving bounds for the row of the next group's last step
    int live_s, live_e, live_d, live_L, live_dir, live_reach, live_left;
};

// The renormalisation takes the minimum over the states that can still lie on a path from the start
// state to the end state: those reached from the start in at most p edges from which the end is at
// most L - p edges away, p being the number of frames consumed by the row in question.  Without
// this the minimum of a tightly constrained sequence sits at states that lag behind (cheap to stay
// in, but too far from the end to matter), the states that carry the posterior mass are hundreds
// of units above it, and their rows lose that much of float's precision (130 sequences of 991 states
// over 1030 frames: posterior error 8.2e-5 before, 2.4e-5 with it).  Any offset is a valid one: the
// states left out just end up below zero.
// live_window: the steps whose row can hold state x on a complete path, as the first such step and the
// number of further ones.  Known for automata whose edges never lower the state number (the
// preparation then leaves the largest rise in the meta record, see min_steps); otherwise every
// state counts in every step.  Two registers per state, and nothing for the scalar unit to carry
// through the time loop.
struct LiveWindow { int first; unsigned more; };
__device__ __forceinline__ LiveWindow live_window(const SeqMeta& m, const int dir, const int x) {
    const int d = m.pad >> 8, L = m.L;
    LiveWindow all = { 0, 0x7fffffffu }, never = { 0x7fffffff, 0u };
    if (d <= 0) return all;
    if (x < m.start_local || x > m.end_local) return never;
    const int plo = (x - m.start_local + d - 1) / d, phi = L - (m.end_local - x + d - 1) / d;    // frames consumed: plo <= p <= phi
    // step i produces the row with p = i + 1 (alpha) or p = L - 1 - i (beta)
    const int lo = max(0, dir ? L - 1 - phi : plo - 1), hi = dir ? L - 1 - plo : phi - 1;
    if (hi < lo) return never;
    LiveWindow w = { lo, (unsigned)(hi - lo) };
    return w;
}
__device__ __forceinline__ bool is_live(const LiveWindow& w, const int i) { return (unsigned)(i - w.first) <= w.more; }
// The same set seen from a step: the state numbers [lo, lo + span] that are live in the row it produces.
// The instance with fifteen compute waves asks this way: it has no registers left for a window per state
// (5 % of its time, measured), while scalar registers and the scalar unit are idle there; for the other
// instances it is the other way round (a sequence of scalar operations in front of the wave minimum costs
// a latency-bound step 4-6 %).
template <int THREADS> struct LiveByStates { static constexpr bool value = THREADS == REC_THREADS_BIG; };
struct LiveStates { int lo; unsigned span; };
__device__ __forceinline__ LiveStates live_interval(const RecCursor& cur, const int reach, const int left) {
    const int hi = min(cur.live_e, reach), lo = max(cur.live_s, left);
    LiveStates r = { lo, hi >= lo ? (unsigned)(hi - lo) : 0u };
    return r;
}
__device__ __forceinline__ LiveStates live_states(const RecCursor& cur, const int i) {
    if (cur.live_d <= 0) { LiveStates all = { 0, 0x7fffffffu }; return all; }
    const long long p = cur.live_dir ? cur.live_L - 1 - i : i + 1;      // frames consumed by the row step i produces
    const long long reach = cur.live_s + p * cur.live_d, left = cur.live_e - (cur.live_L - p) * cur.live_d;
    return live_interval(cur, (int)(reach < cur.live_e ? reach : cur.live_e), (int)(left > cur.live_s ? left : cur.live_s));
}
__device__ __forceinline__ bool is_live(const LiveStates& l, const int s) { return (unsigned)(s - l.lo) <= l.span; }

// End of a step: the per-frame barrier and, every PUBLISH steps, the progress counter.  Stores
// complete in issue order, so "at most PUBLISH of this wave's stores are still in flight" means
// that every row older than PUBLISH steps has been written through (a wave issues at least one
// store per step or none at all); publishing that older count never drains the store queue, which
// would cost several microseconds per publication while the dense write saturates the memory.
template <bool SYNC>
__device__ __forceinline__ void step_end(const int i, RecCursor& cur) {
#ifdef I6_TRACE
    if (threadIdx.x == 0 && (i % 50) == 0 && (blockIdx.x < 2 || blockIdx.x >= gridDim.x - 2))
    {
        g_trace[64 + (blockIdx.x < 2 ? blockIdx.x : 2 + (blockIdx.x & 1)) * 64 + i / 50] = wall_clock64();
        g_trace[64 + (blockIdx.x < 2 ? blockIdx.x : 2 + (blockIdx.x & 1)) * 64 + 32 + i / 50] = clock64();
    }
#endif
    static_assert(PUBLISH == 32, "the wait count below is PUBLISH");
    const bool last = i + 1 == cur.nsteps;
    const bool pub = SYNC && (((i + 1) % PUBLISH) == 0 || last);
    if (pub) {
        if (last) wait_stores();
        else asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
    }
#ifdef I6_TRACE
    const bool tr_ = blockIdx.x == 0 && i >= 400 && i < 432 && (threadIdx.x & 63) == 0 && (threadIdx.x == 0 || threadIdx.x == 320);
    if (tr_) g_trace[3200 + (threadIdx.x ? 64 : 0) + 2 * (i - 400)] = wall_clock64();
    lds_barrier();
    if (tr_) g_trace[3200 + (threadIdx.x ? 64 : 0) + 2 * (i - 400) + 1] = wall_clock64();
#else
    lds_barrier();
#endif
    // (not after the loader wave has given up waiting for a strip of the gather: rows computed from
    // then on may be built on scores that were not there yet, and whoever waits for them must run into
    // its own limit and write NaN rather than use them.  The loader says so in LDS: a flag in memory
    // would cost this wave a round trip, and the other waves a wait at the next barrier, every time.)
    if (pub && threadIdx.x == 0 && !*cur.gave_up) store_agent(cur.progress, last ? i + 2 : i + 2 - PUBLISH);
}

// One frame for the states tid + j*THREADS: predecessor values and staged emission scores from
// LDS, log-sum-exp (base 2) in a fixed order, result to the other LDS buffer and the workspace.
template <typename ST> __device__ __forceinline__ ST state_min(ST a, ST b) { return b < a ? b : a; }
// minimum as one instruction; of a number and a NaN, the number
__device__ __forceinline__ float num_min(float a, float b) { return __builtin_fminf(a, b); }
__device__ __forceinline__ double num_min(double a, double b) { return __builtin_fmin(a, b); }

// Value of a state after a frame, from the scores v[k] of its KT candidates (predecessor value +
// edge weight + emission score): -log2 of the sum of the 2^-v[k], less the renormalisation `pend`.
// Two candidates (left-to-right automata: stay or advance): min - log2(1 + 2^-|v0 - v1|), one exp2
// instead of two and no comparison; inf - inf gives NaN, which the maximum with 0 replaces (the
// result is then inf - 1 = inf, as it must be for a state none of whose predecessors is alive).
template <int KT, typename ST, bool PEND>
__device__ __forceinline__ ST state_value(const ST (&v)[KT], const float pend) {
    if (KT == 2) {
        const ST mn = num_min(v[0], v[1]);
        const float d = __builtin_fmaxf(__builtin_fabsf((float)(v[0] - v[1])), 0.f);
        const float l = __builtin_amdgcn_logf(1.f + __builtin_amdgcn_exp2f(-d));
        return (PEND ? mn - (ST)pend : mn) - (ST)l;
    }
    ST mn = v[0];
#pragma unroll
    for (int k = 1; k < KT; k++) mn = num_min(mn, v[k]);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < KT; k++) sum += __builtin_amdgcn_exp2f((float)(mn - v[k]));
    // sum is in [1, KT] whenever mn is finite: the raw log2 needs no range handling.  With every
    // candidate at +inf the differences are NaN and so is the result: the minimum with +inf, which
    // returns the operand that is a number, turns it into the +inf it must be.
    return num_min((PEND ? mn - (ST)pend : mn) - (ST)__builtin_amdgcn_logf(sum), (ST)INF_F);
}


// ST is the type of the state vector in LDS: float, or double for sequences whose alignment is so
// constrained that the states carrying the posterior mass sit far from the frame minimum (their
// values would lose precision in float, frame after frame).  exp2 / log2 always work in float on
// differences, which are small; rows go to the workspace as float either way.
// NJ: how many of the J rounds (states tid + j*THREADS) hold a state for this wave
template <bool SYNC, int THREADS, int J, int KT, typename ST, int NJ>
__device__ __forceinline__ void recurse_step(const int i, const int SP, const char* stc, ST* stn,
                                             const char* amc, float* wmin,
                                             const unsigned (&eo)[J][KT], const unsigned (&es)[J][KT],
                                             const float (&ew)[J][KT], const LiveWindow (&lw)[J], RecCursor& cur) {
    constexpr int NW = THREADS / 64;
    const int tid = threadIdx.x;
    float pend = 0.f;
    if (cur.pending) {
        float mn = wmin[0];
#pragma unroll
        for (int w = 1; w < NW; w++) mn = fminf(mn, wmin[w]);
        pend = mn == INF_F ? 0.f : mn;
        cur.c += (double)pend;
    }
    float rj[NJ > 0 ? NJ : 1];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int s = tid + j * THREADS;
        ST v[KT];
#pragma unroll
        for (int k = 0; k < KT; k++) v[k] = *(const ST*)(stc + eo[j][k]) + (ST)(ew[j][k] + *(const float*)(amc + es[j][k]));
        const ST r = state_value<KT, ST, true>(v, pend);
        stn[s] = r;
        if (s < SP) store_x<SYNC>(cur.wp + s, (float)r);
        rj[j] = (float)r;
    }
    if (tid == 0) store_x<SYNC>(cur.op, cur.c);
    cur.wp += cur.wstep; cur.op += cur.ostep;
    cur.pending = (i % RENORM) == RENORM - 1;
    if (cur.pending) {
        float rmin = INF_F;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const bool live = LiveByStates<THREADS>::value ? is_live(live_states(cur, i), tid + j * THREADS) : is_live(lw[j], i);
            rmin = fminf(rmin, live ? rj[j] : INF_F);
        }
        rmin = wave_min_dpp(rmin);
        if ((tid & 63) == 63) wmin[tid >> 6] = rmin;
    }
    step_end<SYNC>(i, cur);
}

// One frame of a group of RENORM frames, its place in the group known at compile time: FIRST takes
// up the renormalisation the previous group asked for (and writes the offsets of all rows of the
// group, which share it: lanes 0..RENORM-1 of the first wave, one store each), LAST leaves the
// wave's minimum for the next group.  The steps between them are nothing but the arithmetic, the
// row store and the barrier (which the caller issues): the recursion is bound by the number of
// instructions a SIMD has to issue per frame for the waves it holds.
template <bool SYNC, int THREADS, int J, int KT, typename ST, int NJ, bool FIRST, bool LAST>
__device__ __forceinline__ void recurse_step_in_group(const int i, const int SP, const char* stc, ST* stn, const char* amc, float* wmin,
                                                      const unsigned (&eo)[J][KT], const unsigned (&es)[J][KT],
                                                      const float (&ew)[J][KT], const LiveWindow (&lw)[J], RecCursor& cur) {
    constexpr int NW = THREADS / 64;
    const int tid = threadIdx.x;
    float pend = 0.f;
    if (FIRST) {
        float mn = wmin[0];
#pragma unroll
        for (int w = 1; w < NW; w++) mn = fminf(mn, wmin[w]);
        pend = mn == INF_F ? 0.f : mn;
        cur.c += (double)pend;
        if (tid < RENORM) store_x<SYNC>(cur.op + tid * cur.ostep, cur.c);
        cur.op += RENORM * cur.ostep;
    }
    float rmin = INF_F;
    LiveStates states = { 0, 0u };
    if (LAST && LiveByStates<THREADS>::value) {
        // (the two bounds move by RENORM frames from one group to the next; a sequence long enough for them to leave the
        // range of int has had its live_d set to 0 by recurse_init)
        states = live_interval(cur, cur.live_reach, cur.live_left);
        const int inc = (cur.live_dir ? -RENORM : RENORM) * cur.live_d;
        cur.live_reach += inc; cur.live_left += inc;
    }
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int s = tid + j * THREADS;
        ST v[KT];
#pragma unroll
        for (int k = 0; k < KT; k++) v[k] = *(const ST*)(stc + eo[j][k]) + (ST)(ew[j][k] + *(const float*)(amc + es[j][k]));
        const ST r = state_value<KT, ST, FIRST>(v, pend);
        stn[s] = r;
        if (s < SP) store_x<SYNC>(cur.wp + s, (float)r);
        if (LAST) rmin = fminf(rmin, (LiveByStates<THREADS>::value ? is_live(states, s) : is_live(lw[j], i)) ? (float)r : INF_F);
    }
    cur.wp += cur.wstep;
    if (LAST) {
        rmin = wave_min_dpp(rmin);
        if ((tid & 63) == 63) wmin[tid >> 6] = rmin;
    }
}

// all steps of a wave that has states in NJ of its J rounds
template <bool SYNC, int THREADS, int J, int KT, typename ST, int NJ>
__device__ __forceinline__ void recurse_time_loop(const int SP, ST* st0, ST* st1, const float* am0, const float* am1, float* wmin,
                                                  const unsigned (&eo)[J][KT], const unsigned (&es)[J][KT],
                                                  const float (&ew)[J][KT], const LiveWindow (&lw)[J], RecCursor& cur) {
    static_assert(RENORM == 8 && PUBLISH % RENORM == 0, "shape of a group of steps");
    const char* c0 = (const char*)st0; const char* c1 = (const char*)st1;
    const char* a0 = (const char*)am0; const char* a1 = (const char*)am1;
    int i = 0;
    // whole groups of RENORM steps, as long as the last step of the sequence is not among them
    for (; i + RENORM < cur.nsteps; i += RENORM) {
#ifdef I6_TRACE
        if (threadIdx.x == 0 && (i % 48) == 0 && (blockIdx.x < 2 || blockIdx.x >= gridDim.x - 2)) {
            g_trace[64 + (blockIdx.x < 2 ? blockIdx.x : 2 + (blockIdx.x & 1)) * 64 + i / 48] = wall_clock64();
            g_trace[64 + (blockIdx.x < 2 ? blockIdx.x : 2 + (blockIdx.x & 1)) * 64 + 32 + i / 48] = clock64();
        }
#endif
        recurse_step_in_group<SYNC, THREADS, J, KT, ST, NJ, true, false>(i, SP, c0, st1, a0, wmin, eo, es, ew, lw, cur);
        lds_barrier();
        recurse_step_in_group<SYNC, THREADS, J, KT, ST, NJ, false, false>(i, SP, c1, st0, a1, wmin, eo, es, ew, lw, cur);
        lds_barrier();
        for (int r = 0; r < (RENORM - 4) / 2; r++) {
            recurse_step_in_group<SYNC, THREADS, J, KT, ST, NJ, false, false>(i, SP, c0, st1, a0, wmin, eo, es, ew, lw, cur);
            lds_barrier();
            recurse_step_in_group<SYNC, THREADS, J, KT, ST, NJ, false, false>(i, SP, c1, st0, a1, wmin, eo, es, ew, lw, cur);
            lds_barrier();
        }
        recurse_step_in_group<SYNC, THREADS, J, KT, ST, NJ, false, false>(i, SP, c0, st1, a0, wmin, eo, es, ew, lw, cur);
        lds_barrier();
        recurse_step_in_group<SYNC, THREADS, J, KT, ST, NJ, false, true>(i + RENORM - 1, SP, c1, st0, a1, wmin, eo, es, ew, lw, cur);
        // as step_end for the step i + RENORM - 1, which is never the last one
        const bool pub = SYNC && ((i + RENORM) % PUBLISH) == 0;
        static_assert(PUBLISH == 32, "the wait count below is PUBLISH");
        if (pub) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
        lds_barrier();
        if (pub && threadIdx.x == 0 && !*cur.gave_up) store_agent(cur.progress, i + RENORM + 1 - PUBLISH);
    }
    cur.pending = i > 0;
    // the rest, at most RENORM steps, the last one among them
    for (; i < cur.nsteps; i += 2) {
        recurse_step<SYNC, THREADS, J, KT, ST, NJ>(i, SP, c0, st1, a0, wmin, eo, es, ew, lw, cur);
        if (i + 1 < cur.nsteps)
            recurse_step<SYNC, THREADS, J, KT, ST, NJ>(i + 1, SP, c1, st0, a1, wmin, eo, es, ew, lw, cur);
    }
}

// common prologue of the compute waves: initial state vector, row 0 of the workspace, cursor
template <bool SYNC, int THREADS, typename ST>
__device__ __forceinline__ void recurse_init(const RecArgs& a, const SeqMeta& m, const int b, const int dir, const int SCAP,
                                             ST* st0, ST* st1, float* wmin, RecCursor& cur) {
    const int tid = threadIdx.x;
    const int L = m.L, SP = m.SP, T = a.T;
    const long long soff = state_off(m.edge_begin, b);
    float* ws = (dir ? a.beta : a.alpha) + (size_t)T * soff;
    double* offs = (dir ? a.offB : a.offA) + (size_t)b * T;
    const int init_state = dir ? m.end_local : m.start_local;
    const int row0 = dir ? L - 1 : 0;
    for (int s = tid; s < SCAP; s += THREADS) {
        const float v = s == init_state ? 0.f : INF_F;
        st0[s] = v;
        st1[s] = INF_F;
        if (s < SP) store_x<SYNC>(&ws[(size_t)row0 * SP + s], v);
    }
    if (tid < 16) { st0[SCAP + tid] = INF_F; st1[SCAP + tid] = INF_F; }
    if (tid == 0) store_x<SYNC>(&offs[row0], 0.0);
    // step i consumes frame f(i) = i (alpha) or L-1-i (beta) and produces the row stored for
    // frame f(i)+1 (alpha) or f(i)-1 (beta); L-1 steps in all
    cur.wstep = dir ? -(long long)SP : (long long)SP;
    cur.wp = ws + (size_t)row0 * SP + cur.wstep;
    cur.ostep = dir ? -1 : 1;
    cur.op = offs + row0 + cur.ostep;
    cur.c = 0.0;
    cur.pending = false;
    cur.progress = a.sync + SYNC_HDR + 2 * b + dir;
    cur.gave_up = rec_gave_up(wmin);
    cur.nsteps = L - 1;
    cur.live_s = m.start_local; cur.live_e = m.end_local; cur.live_L = L; cur.live_dir = dir;
    cur.live_d = (long long)(m.pad >> 8) * L < (1 << 30) ? m.pad >> 8 : 0;
    if (cur.live_d > 0) {
        const int p = dir ? L - RENORM : RENORM;       // frames consumed by the row of step RENORM - 1, the first to ask
        cur.live_reach = cur.live_s + p * cur.live_d; cur.live_left = cur.live_e - (L - p) * cur.live_d;
    } else {
        cur.live_s = 0; cur.live_e = 0x7fffffff; cur.live_reach = 0x7fffffff; cur.live_left = 0;
    }
    if (SYNC) wait_stores();
    lds_barrier();
    if (SYNC && tid == 0) store_agent(cur.progress, 1);      // the initial row is out
}

template <bool SYNC, int THREADS, int J, int KT, typename ST>
__device__ __forceinline__ void recurse_compute(const RecArgs& a, const SeqMeta& m, const int b, const int dir,
                                                ST* st0, ST* st1,
                                                const float* am0, const float* am1,
                                                float* wmin) {
    constexpr int SCAP = THREADS * J;
    const int tid = threadIdx.x;
    const int SP = m.SP;
    const long long soff = state_off(m.edge_begin, b);
    const uint2* ell = (dir ? a.ellB : a.ellA) + (size_t)KMAX * soff;
    const int K = dir ? m.Kout : m.Kin;

    // edges of my states -> registers, as LDS byte offsets of the other state / the emission slot
    unsigned eo[J][KT], es[J][KT];
    float ew[J][KT];
#pragma unroll
    for (int j = 0; j < J; j++) {
        const int s = tid + j * THREADS;
#pragma unroll
        for (int k = 0; k < KT; k++) {
            uint2 r = make_uint2(NO_STATE, 0u);
            if (k < K && s < SP) r = ell[(size_t)k * SP + s];
            unsigned other = r.x & 0xFFFFu;
            if (other == NO_STATE) other = SCAP;          // LDS cell that always holds +inf
            eo[j][k] = other * (unsigned)sizeof(ST);
            es[j][k] = (r.x >> 16) * 4u;
            ew[j][k] = __uint_as_float(r.y);
        }
    }
    LiveWindow lw[J];
#pragma unroll
    for (int j = 0; j < J; j++) {
        if (LiveByStates<THREADS>::value) { lw[j].first = 0; lw[j].more = 0u; }      // not used: see live_states
        else lw[j] = live_window(m, dir, tid + j * THREADS);
    }
    if (tid < THREADS / 64) wmin[tid] = INF_F;
    RecCursor cur;
    recurse_init<SYNC, THREADS, ST>(a, m, b, dir, SCAP, st0, st1, wmin, cur);
    // Rounds of this wave that hold a state at all (the cells of the others keep the +inf of the
    // start-up); the time loop is instantiated for that number, so that the LDS reads of all its
    // rounds are issued together.  Waves without a state leave: they would only compete with the
    // others for issue slots on their SIMD, and a barrier counts the waves that are still there.
    // Their entries of wmin keep the +inf written above.
    const int first = tid & ~63;
    const int nj = first >= SP ? 0 : min(J, (SP - first + THREADS - 1) / THREADS);
    if (nj == 0) return;
    // (only in the instance for small batches: the one of which two workgroups share a compute unit
    // has no registers to spare for more loop bodies)
    constexpr bool PER_ROUND = THREADS == REC_THREADS || THREADS == REC_THREADS_BIG;
    if (!PER_ROUND) recurse_time_loop<SYNC, THREADS, J, KT, ST, J>(SP, st0, st1, am0, am1, wmin, eo, es, ew, lw, cur);
    else if (J == 1 || nj == 1) recurse_time_loop<SYNC, THREADS, J, KT, ST, 1>(SP, st0, st1, am0, am1, wmin, eo, es, ew, lw, cur);
    else if (nj == 2) recurse_time_loop<SYNC, THREADS, J, KT, ST, (J >= 2 ? 2 : 1)>(SP, st0, st1, am0, am1, wmin, eo, es, ew, lw, cur);
    else if (nj == 3) recurse_time_loop<SYNC, THREADS, J, KT, ST, (J >= 3 ? 3 : 1)>(SP, st0, st1, am0, am1, wmin, eo, es, ew, lw, cur);
    else recurse_time_loop<SYNC, THREADS, J, KT, ST, J>(SP, st0, st1, am0, am1, wmin, eo, es, ew, lw, cur);
}

// Fallback for the largest sequences: same arithmetic, edge tables re-read from memory each frame
// instead of living in registers.
template <bool SYNC, int THREADS, typename ST>
__device__ __forceinline__ void recurse_compute_generic(const RecArgs& a, const SeqMeta& m, const int b, const int dir,
                                                        ST* st0, ST* st1,
                                                        const float* am0, const float* am1,
                                                        float* wmin, const int SCAP) {
    constexpr int NW = THREADS / 64;
    const int tid = threadIdx.x;
    const int SP = m.SP;
    const long long soff = state_off(m.edge_begin, b);
    const uint2* ell = (dir ? a.ellB : a.ellA) + (size_t)KMAX * soff;
    const int K = dir ? m.Kout : m.Kin;
    RecCursor cur;
    recurse_init<SYNC, THREADS, ST>(a, m, b, dir, SCAP, st0, st1, wmin, cur);
    ST* stc = st0; ST* stn = st1;
    const float* amc = am0; const float* amn = am1;
    for (int i = 0; i < cur.nsteps; i++) {
        float pend = 0.f;
        if (cur.pending) {
            float mn = wmin[0];
#pragma unroll
            for (int w = 1; w < NW; w++) mn = fminf(mn, wmin[w]);
            pend = mn == INF_F ? 0.f : mn;
            cur.c += (double)pend;
        }
        float rmin = INF_F;
        const bool want_min = (i % RENORM) == RENORM - 1;       // over the states that still matter, see live_window
        if (K > KMAX) {
            // degree beyond the unrolled body: two passes over the state's table column
            for (int s = tid; s < SP; s += THREADS) {
                auto value = [&](int k) -> ST {
                    const uint2 r = ell[(size_t)k * SP + s];
                    const unsigned other = r.x & 0xFFFFu;
                    return other == NO_STATE ? (ST)INF_F : stc[other] + (ST)(__uint_as_float(r.y) + amc[r.x >> 16]);
                };
                ST mn = (ST)INF_F;
                for (int k = 0; k < K; k++) mn = state_min(mn, value(k));
                float sum = 0.f;
                for (int k = 0; k < K; k++) sum += __builtin_amdgcn_exp2f((float)(mn - value(k)));
                const ST r = mn == (ST)INF_F ? (ST)INF_F : (mn - (ST)pend) - (ST)__builtin_amdgcn_logf(sum);
                stn[s] = r;
                store_x<SYNC>(cur.wp + s, (float)r);
                if (want_min && is_live(live_window(m, dir, s), i)) rmin = fminf(rmin, (float)r);
            }
        } else
        for (int s = tid; s < SP; s += THREADS) {
            ST v[KMAX];
            ST mn = (ST)INF_F;
#pragma unroll
            for (int k = 0; k < KMAX; k++) {
                v[k] = (ST)INF_F;
                if (k < K) {
                    const uint2 r = ell[(size_t)k * SP + s];
                    const unsigned other = r.x & 0xFFFFu;
                    if (other != NO_STATE) v[k] = stc[other] + (ST)(__uint_as_float(r.y) + amc[r.x >> 16]);
                    mn = state_min(mn, v[k]);
                }
            }
            float sum = 0.f;
#pragma unroll
            for (int k = 0; k < KMAX; k++) sum += __builtin_amdgcn_exp2f((float)(mn - v[k]));
            const ST r = mn == (ST)INF_F ? (ST)INF_F : (mn - (ST)pend) - (ST)__builtin_amdgcn_logf(sum);
            stn[s] = r;
            store_x<SYNC>(cur.wp + s, (float)r);
            if (want_min && is_live(live_window(m, dir, s), i)) rmin = fminf(rmin, (float)r);
        }
        if (tid == 0) store_x<SYNC>(cur.op, cur.c);
        cur.wp += cur.wstep; cur.op += cur.ostep;
        cur.pending = (i % RENORM) == RENORM - 1;
        if (cur.pending) {
            rmin = wave_min_dpp(rmin);
            if ((tid & 63) == 63) wmin[tid >> 6] = rmin;
        }
        step_end<SYNC>(i, cur);
        ST* t_ = stc; stc = stn; stn = t_;
        const float* u_ = amc; amc = amn; amn = u_;
    }
}

// Loader wave: keeps the compact emission rows of the next P frames in flight (registers, 8-byte
// pieces) and drops the row of frame f(i+1) into the idle LDS buffer during step i.  It issues
// no global stores, so its wait counts stay exact.  With SYNC it first makes sure the gather
// kernel has finished the strip a row belongs to.
template <bool SYNC, int THREADS, int JL, int P>
__device__ __forceinline__ void recurse_load(const RecArgs& a, const SeqMeta& m, const int b, const int dir,
                                             float* am0, float* am1, int* gave_up) {
    typedef unsigned long long u64;
    const int lane = threadIdx.x - THREADS;
    const int L = m.L, DP = m.DP, T = a.T;
    const long long goff = slot_off(m.edge_begin, b);
    const float* G = a.gtab + (size_t)T * goff;
    const int nsteps = L - 1;
    // My pieces of a row, lane + jl*64, come through buffer loads: the resource describes the one row (its address, its
    // length in bytes), the lane's offset 8 * lane + 512 * jl is checked against that length by the hardware, and a piece
    // past the end of the row comes back as zero without touching memory (it lands in LDS cells no edge refers to).
    // One vector register addresses all pieces of all rows, where global loads clamped to the row took a 64-bit address
    // per piece (with 32 pieces per lane those alone filled half of the register budget of the largest instance, which
    // spilled); reading on past the row's end instead costs the large-automaton instance 3 % (its rows are read
    // from the memory side while the gather is still writing).
    const int lane8 = lane * 8;
    auto piece = [&](const u64* row, int jl) -> u64 {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)row, 0, DP * 4, 0x00020000);
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(rs, lane8 + jl * 512, 0, SYNC ? 16 : 0);      // (16: sc1, the agent-scope load of load_agent)
        return ((u64)v[1] << 32) | v[0];
    };
    int* abort_flag = a.sync;
    const int* gflag = a.sync + SYNC_HDR + 2 * a.B + (size_t)b * ((T + TG - 1) / TG);
    const int nstrip = (L + TG - 1) / TG;
    int strip_ok = -1;                  // strip known to be complete
    int ahead_strip = -1, ahead_val = 0;   // flag of the strip after it, loaded while strip_ok is being consumed
    // row consumed by step i (clamped to the steps that exist); makes sure its strip is complete.
    // The flag of the following strip is requested a strip ahead, so that in the steady state the
    // loader never sits in a memory round trip while the compute waves wait at the barrier.
    auto rowp = [&](int i) -> const u64* {
        const int ic = min(i, nsteps - 1);
        const int f = dir ? L - 1 - ic : ic;
        if (SYNC && f / TG != strip_ok) {
            const int j = f / TG;
            if (!(j == ahead_strip && ahead_val >= 1) && !spin_until_ge(gflag + j, 1, abort_flag)) *gave_up = 1;
            strip_ok = j;
            const int jn = dir ? j - 1 : j + 1;
            ahead_strip = -1;
            if (jn >= 0 && jn < nstrip) { ahead_strip = jn; ahead_val = load_agent(gflag + jn); }
        }
        return (const u64*)(G + (size_t)f * DP);
    };
    u64 g[P][JL];
    if (nsteps > 0) {
        const u64* r0 = rowp(0);
#pragma unroll
        for (int jl = 0; jl < JL; jl++) ((u64*)am0)[lane + jl * 64] = piece(r0, jl);
#pragma unroll
        for (int p = 0; p < P; p++) {
            const u64* rp = rowp(1 + p);
#pragma unroll
            for (int jl = 0; jl < JL; jl++) g[p][jl] = piece(rp, jl);
        }
    }
    lds_barrier();      // pairs with the barrier at the end of recurse_init
    u64* amn = (u64*)am1; u64* amc = (u64*)am0;
    int i0 = 0;
    for (; i0 + P <= nsteps; i0 += P) {
#pragma unroll
        for (int q = 0; q < P; q++) {
            const u64* nxt = rowp(i0 + q + 1 + P);
#pragma unroll
            for (int jl = 0; jl < JL; jl++) {
                amn[lane + jl * 64] = g[q][jl];
                g[q][jl] = piece(nxt, jl);
            }
#ifdef I6_TRACE
            { const int i_ = i0 + q; const bool tr_ = blockIdx.x == 0 && i_ >= 400 && i_ < 432 && lane == 0;
              if (tr_) g_trace[3200 + 128 + 2 * (i_ - 400)] = wall_clock64();
              lds_barrier();
              if (tr_) g_trace[3200 + 128 + 2 * (i_ - 400) + 1] = wall_clock64(); }
#else
            lds_barrier();
#endif
            u64* t_ = amc; amc = amn; amn = t_;
        }
    }
#pragma unroll
    for (int q = 0; q < P; q++) {
        if (i0 + q < nsteps) {
#pragma unroll
            for (int jl = 0; jl < JL; jl++) amn[lane + jl * 64] = g[q][jl];
            lds_barrier();
            u64* t_ = amc; amc = amn; amn = t_;
        }
    }
}

// REC_THREADS compute threads plus one loader wave per workgroup; grid = 2B.
// DENSE is the instance of which two workgroups fit on a compute unit: eight waves, and at most 96
// registers -- two workgroups are four waves per SIMD, and the rest of the register file is what
// the gate, gather and combine waves need to get onto the unit at all.
// The host picks it when the batch has more workgroups than the device has compute units.  The rarely used large-automaton paths pay for the cap with spills,
// which is why small batches run the uncapped instance.
// LDS of a recursion workgroup, in floats: two emission rows, two state vectors (of doubles in
// the uncapped instance, see recurse_step), per-wave minima / reduction scratch, a flag.
constexpr int REC_LDS_FLOATS_F32 = 2 * D_MAX + 2 * (S_MAX + 16) + 32 + 8;
static_assert(DENSE_F64_STATES >= 4 * REC_THREADS_DENSE, "the second size class of the dense instance fits in double");
static_assert(2 * (DENSE_F64_STATES + 16) * 2 <= 2 * (S_MAX + 16), "two double vectors fit the float instance's state area");
constexpr int REC_LDS_FLOATS_F64 = 2 * D_MAX + 4 * (S_MAX + 16) + 32 + 8;

// the compute threads' part for one state type; the loader waves do not depend on it
// ONE: whether sequences with one state per thread can arrive here with this state type (they are
// not instantiated otherwise: fewer loop bodies in a kernel give the remaining ones better code)
// MANY: the same for the larger classes and the table-driven fallback
template <bool SYNC, int T_, typename ST, bool ONE, bool MANY = true>
__device__ __forceinline__ void recurse_dispatch(const RecArgs& a, const SeqMeta& m, const int b, const int dir, const int cls,
                                                 ST* st0, ST* st1, const float* am0, const float* am1, float* wmin,
                                                 const int scap_big = S_MAX) {
    const int K = dir ? m.Kout : m.Kin;
    // The loop body is specialised on the number of states per thread and of edge slots per state,
    // so that all LDS reads of a frame are issued back to back; unused slots read the +inf cell.
    constexpr bool F32 = sizeof(ST) == 4;
    if (MANY && K > KMAX) {
        recurse_compute_generic<SYNC, T_, ST>(a, m, b, dir, st0, st1, am0, am1, wmin, scap_big);
    } else if (ONE && cls == 1) {
        if (K <= 2) recurse_compute<SYNC, T_, 1, 2, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else if (K <= 3) recurse_compute<SYNC, T_, 1, 3, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else if (K <= 4) recurse_compute<SYNC, T_, 1, 4, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else if (K <= 6) recurse_compute<SYNC, T_, 1, 6, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else recurse_compute<SYNC, T_, 1, KMAX, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
    } else if (!MANY) {
        return;
    } else if (cls == 2) {
        if (K <= 2) recurse_compute<SYNC, T_, 4, 2, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else if (K <= 3) recurse_compute<SYNC, T_, 4, 3, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else if (K <= 4) recurse_compute<SYNC, T_, 4, 4, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        // (degree 5-8 with at most two states per thread still fits the registers -- CTC automata, whose
        // final states collect five edges: 603 states over 945 frames took 2.3 us per frame through the
        // table-driven loop below)
        else if (m.SP <= 2 * T_ && K <= 6) recurse_compute<SYNC, T_, 2, 6, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else if (m.SP <= 2 * T_) recurse_compute<SYNC, T_, 2, KMAX, ST>(a, m, b, dir, st0, st1, am0, am1, wmin);
        else recurse_compute_generic<SYNC, T_, ST>(a, m, b, dir, st0, st1, am0, am1, wmin, 4 * T_);
    } else {
        recurse_compute_generic<SYNC, T_, ST>(a, m, b, dir, st0, st1, am0, am1, wmin, scap_big);
    }
}

// INST: 0 the instance for small batches, 1 the dense one (two workgroups per compute unit), 2 the one for large automata
template <bool SYNC, int INST>
__device__ __forceinline__ void recurse_workgroup(const RecArgs& a, float* lds) {
    constexpr bool DENSE = INST == 1;
    constexpr int T_ = INST == 1 ? REC_THREADS_DENSE : (INST == 2 ? REC_THREADS_BIG : REC_THREADS);
    // LDS of a workgroup (16-byte aligned): the emission rows first
    float (*amr)[D_MAX] = (float (*)[D_MAX])lds;
    float* stf = lds + 2 * D_MAX;                                        // state vectors, float or double
    float* wmin = stf + (DENSE ? 2 : 4) * (S_MAX + 16);
    int* go_flag = rec_go_flag(wmin);      // wmin doubles as the 32-float scratch of the general path's reductions

    // the recursion is the latency-critical kernel: its waves go first when they share a SIMD with
    // gather or combine waves
    __builtin_amdgcn_s_setprio(3);
#ifdef I6_TRACE
    if (threadIdx.x == 0 && blockIdx.x < 64) g_trace[3000 + blockIdx.x] = trace_cu_key();
#endif
    if (SYNC) {
        // This kernel is started beside the preparation, so that its large workgroups are placed
        // while the machine is still empty: report the placement (see fbw_gate), wait until all
        // preparation workgroups have counted themselves, then drop stale cache lines.
        if (threadIdx.x == 0) {
            atomicAdd(&a.sync[1], 1);
            *go_flag = spin_until_ge(a.sync + 3, a.prep_wgs, a.sync) ? 1 : 0;
            *rec_gave_up(wmin) = 0;
        }
        __syncthreads();
        if (!*go_flag) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");      // (and the acquire half all the reader needs: no write-back of the L2 by every wave)
    }
    const int b = blockIdx.x >> 1, dir = blockIdx.x & 1;
    const SeqMeta m = a.meta[b];
    const int cls = rec_class(m, T_);
    if (cls == -2) {
        const long long soff = state_off(m.edge_begin, b);
        float* rows = (dir ? a.beta : a.alpha) + (size_t)a.T * soff;
        double* offs = (dir ? a.offB : a.offA) + (size_t)b * a.T;
        int* progress = a.sync + SYNC_HDR + 2 * b + dir;
        // the sequence's share of the compact emission table is unused on this path: room for the
        // two double-precision working vectors of each direction, unless T is tiny
        const long long goff = slot_off(m.edge_begin, b);
        if (generic_recurse_f64_room(m, b, a.T))
            generic_recurse_f64<SYNC>(a.gen, m, b, dir, a.T, rows, offs, progress, wmin,
                                      (double*)(a.gtab_rw + (size_t)a.T * goff) + (size_t)dir * 2 * m.SP);
        else
            generic_recurse<SYNC>(a.gen, m, b, dir, a.T, rows, offs, progress, wmin);
        return;
    }
    if (cls <= 0) return;
    if (threadIdx.x >= T_) {
        if (cls == 1 && INST == 2) recurse_load<SYNC, T_, 8, 4>(a, m, b, dir, amr[0], amr[1], rec_gave_up(wmin));
        else if (cls == 1) recurse_load<SYNC, T_, 4, 8>(a, m, b, dir, amr[0], amr[1], rec_gave_up(wmin));
        else if (cls == 2) recurse_load<SYNC, T_, 16, 2>(a, m, b, dir, amr[0], amr[1], rec_gave_up(wmin));
        else recurse_load<SYNC, T_, 32, 1>(a, m, b, dir, amr[0], amr[1], rec_gave_up(wmin));
        return;
    }
    // Double-precision state vectors where float would show in the posteriors.  State values are
    // relative to the frame minimum, and the states that carry the posterior mass can sit a
    // hundred units and more above it; float then loses a little in every frame (a CTC automaton of
    // 116 labels over 764 frames reached 1.05e-4 on the posteriors, 1.2e-5 in double; 1100 states in
    // 1055 frames 1.4e-4; 20 000 frames through 100 states 3e-4).  Up to 256 states -- one wave per
    // SIMD, bound by latency more than by arithmetic -- double costs 7 % of the recursion and is used
    // for sequences with fewer than four frames per state; beyond that it costs 15-20 % and is kept for
    // sequences with fewer than five frames for every three states.  More than I6_FLOAT_FRAMES frames: always
    // (whatever the shape of the automaton, float adds up from frame to frame: CTC automata of 200 labels over
    // 2000 frames 9.7e-5, 177 states over 400 frames 7.1e-5; the sequences this rule alone catches have at most
    // three states for every five frames, i.e. few states per thread, where double costs next to nothing).
    // The dense instance has room in LDS for the small sequences only (and is used for at most 4096
    // frames): batches of more than 128 CTC automata of 110-150 labels over 760-900 frames came out at
    // 8.7e-5 to 9.3e-5 in float.
    const bool small_tight = cls == 1 && m.SP <= 256 && m.L < 4LL * m.S;
    const bool wide = !DENSE && (small_tight || 5LL * m.S > 3LL * m.L || m.L > I6_FLOAT_FRAMES);
    // (there double costs 5-12 % of the recursion time, so only from 256 frames on, where the rounding of float has
    // had time to add up -- but then for every sequence with one state per thread: 140 automata of up to 180 states
    // over up to 400 frames came out at 6.5e-5 in float, 2.4e-5 in double; 140 monophone automata of 250-400 states
    // over 320-400 frames at 8.7e-5 and 3.6e-5; CTC automata of 40-120 states over 150-200 frames are at 1.7e-5
    // in float and would pay 14 us per call)
    if (DENSE && cls == 1 && m.L >= I6_FLOAT_FRAMES && (dir ? m.Kout : m.Kin) <= KMAX) {
        double* st0 = (double*)stf;
        recurse_dispatch<SYNC, T_, double, true, false>(a, m, b, dir, cls, st0, st0 + (T_ + 16), amr[0], amr[1], wmin);
    } else if (DENSE && cls >= 2 && (5LL * m.S > 3LL * m.L || m.L > I6_FLOAT_FRAMES)) {
        // The state area of this instance holds two double vectors of DENSE_F64_STATES + 16 entries (the
        // preparation sends larger sequences of such batches to the general path, see dense_f64_limit).
        // The register cap makes this slow; it is the rare case (hundreds of sequences with thousands
        // of states each and barely more frames than states, or more than I6_FLOAT_FRAMES frames).
        double* st0 = (double*)stf;
        recurse_dispatch<SYNC, T_, double, false, true>(a, m, b, dir, cls, st0, st0 + (DENSE_F64_STATES + 16), amr[0], amr[1], wmin,
                                                        DENSE_F64_STATES);
    } else if (wide) {
        double* st0 = (double*)stf;
        recurse_dispatch<SYNC, T_, double, true>(a, m, b, dir, cls, st0, st0 + (S_MAX + 16), amr[0], amr[1], wmin);
    } else {
        recurse_dispatch<SYNC, T_, float, true>(a, m, b, dir, cls, stf, stf + (S_MAX + 16), amr[0], amr[1], wmin);
    }
}

// RESERVE: in the schedule in which gather and dense write run at the same time the workgroup also
// claims the registers that would let their waves move in beside its own: its nine waves then hold
// 504 (one SIMD) or 336 of a SIMD's 512 registers, as much as three waves per SIMD allow.  Measured
// on the headline workload: with the 142 registers the code needs, 0.575 ms per call; with 168,
// 0.553.  Only for batches that leave half of the compute units without a recursion workgroup:
// 256-thread workgroups need room on every SIMD, and with one of these on every unit the gather
// would find none anywhere.
template <bool SYNC, bool RESERVE = false>
__global__ __launch_bounds__(REC_BLOCK) void fbw_recurse(RecArgs a) {
    __shared__ __attribute__((aligned(16))) float lds[REC_LDS_FLOATS_F64];
    if (RESERVE) asm volatile("v_mov_b32 v167, 0" ::: "v167");
    recurse_workgroup<SYNC, 0>(a, lds);
#ifdef I6_TRACE
    __syncthreads();
    if (threadIdx.x == 0 && blockIdx.x < 64) g_trace[3000 + blockIdx.x] = 1;
#endif
}
// The dense instance takes its LDS as dynamic shared memory (REC_LDS_FLOATS_F32 floats): with the
// size known at compile time the compiler sees that at most two workgroups fit on a unit anyway
// and ignores the register cap, and two workgroups then fill the register file.
// (The cap of 96 registers is for the schedule in which gather and dense write run beside this kernel and need room on
// its compute units; stage after stage -- the schedule the library chooses for such batches -- two workgroups have the
// register file to themselves, four waves per SIMD with 128 registers each, and nothing spills inside the time loops.)
template <bool SYNC>
__global__ __launch_bounds__(REC_BLOCK_DENSE, SYNC ? 5 : 4) void fbw_recurse_dense(RecArgs a) {
    extern __shared__ __attribute__((aligned(16))) float dyn_lds[];
    recurse_workgroup<SYNC, 1>(a, dyn_lds);
}
// Sixteen waves of at most 128 registers: the workgroup has its compute unit's register file to itself
// without asking (see RESERVE above).
template <bool SYNC>
__global__ __launch_bounds__(REC_BLOCK_BIG) void fbw_recurse_big(RecArgs a) {
    __shared__ __attribute__((aligned(16))) float lds[REC_LDS_FLOATS_F64];
    recurse_workgroup<SYNC, 2>(a, lds);
}

// ---------------------------------------------------------------------------------------------
// stage 4: combine.  One workgroup per (strip of TC frames, sequence).  The F-wide row image
// lives in LDS: its non-hole positions are the same for every frame of a sequence, so it is
// filled once and only those positions are rewritten per frame before the row is streamed out.
// ---------------------------------------------------------------------------------------------
struct CombArgs {
    GenArgs gen;
    int T, B, F, out_mode;
    const SeqMeta* meta; const uint4* crec; const int* cbegin; const int* demis;
    const float* alpha; const float* beta; const float* gtab; const double* offA; const double* offB;
    float* out; float* sum_output;
    long long ost_t, ost_b;      // element strides of out over frames and sequences
    int* sync;
    int tile_w;                  // 0: the row image holds the whole row; else its width in floats (a multiple of 32), see finish_row
    int direct_only;             // beside fbw_flat: only the sequences that kernel leaves to this one (flat_direct)
    int small_elsewhere = 0;     // the sequences of comb_small() are written by the SMALL instance of this kernel, launched beside this one
    int pad_rows = 0;            // the general instance also writes the rows of frames >= seq_len (no fbw_padfill in this call)
    int batch_frames = 0;        // SMALL instance: the LDS of the launch holds COMB_BATCH row images and staging areas (comb_batch_lds_bytes)
};

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float float4a __attribute__((ext_vector_type(4)));

// Which kernel writes the rows t < seq_len of a sequence when the dense tensor goes out in flat
// spans (fbw_flat): that kernel itself for sequences small enough for its register-resident
// posterior jobs, fbw_combine (row by row, started beside it with direct_only set) for the larger
// ones and for those on the general path.  Sequences with a reported problem or without edges have
// constant rows, which the write jobs of fbw_flat produce by themselves.
constexpr int COMB_FAST_EDGES = 1024, COMB_FAST_SLOTS = 512;
// (fbw_flat: up to COMB_FAST_* everything of a thread stays in registers over the frames of a job; up to
// FLAT_* the edges are taken in pieces of COMB_FAST_EDGES per frame, their scores parked in the staging area)
constexpr int FLAT_EDGES = 2048, FLAT_SLOTS = 1024;
__device__ __forceinline__ bool flat_fast(const SeqMeta& m) {
    return seq_error(m) == 0 && m.n_edges > 0 && m.L > 0 && m.n_edges <= FLAT_EDGES && m.D <= FLAT_SLOTS;
}
__device__ __forceinline__ bool flat_direct(const SeqMeta& m) {
    return seq_error(m) >= 0 && m.n_edges > 0 && m.L > 0 && !flat_fast(m);
}

// Row streaming.  Rows start at arbitrary 4-byte offsets (F need not be a multiple of 32), so the
// row is addressed from the 128-byte line boundary below its start: chunk c covers floats
// [4c, 4c+4) counted from that boundary, every wave store starts on a line boundary, and only the
// chunks cut by the row's ends fall back to scalar stores.  The line-aligned chunks go out as
// non-temporal stores: the tensor is written once and never read here, and keeping it out of the
// caches measured faster for the whole call (I6_NT=0 switches to plain stores).
#ifndef I6_NT
#define I6_NT 1
#endif
#if I6_NT
#define I6_ROW_STORE(v, p) __builtin_nontemporal_store(v, p)
#else
#define I6_ROW_STORE(v, p) (*(p) = (v))
#endif
__device__ __forceinline__ int row_misalign(const float* row) { return (int)(((uintptr_t)row >> 2) & 31); }

__device__ inline void stream_const_row(float* row, int F, float v) {
    const int a = row_misalign(row);
    float* base = row - a;
    const float4a c = {v, v, v, v};
    const int ch_lo = (a + 3) >> 2, ch_hi = (a + F) >> 2;      // chunks that lie completely inside the row
    for (int ch = threadIdx.x; ch < ch_hi; ch += COMB_THREADS)
        if (ch >= ch_lo) I6_ROW_STORE(c, (float4a*)(base + 4 * ch));
    if (threadIdx.x < 8) {                                      // the floats of the two cut chunks
        const int i = threadIdx.x < 4 ? 4 * (ch_lo - 1) + threadIdx.x : 4 * ch_hi + threadIdx.x - 4;
        if (i >= a && i < a + F && (i < 4 * ch_lo || i >= 4 * ch_hi)) base[i] = v;
    }
}

// image[a + f] holds column f of the row; a = row_misalign(row)
__device__ inline void stream_image_row(float* row, int F, const float4a* lds4, const float* image) {
    const int a = row_misalign(row);
    float* base = row - a;
    const int ch_lo = (a + 3) >> 2, ch_hi = (a + F) >> 2;
    constexpr int U = 4;                                        // LDS reads in flight per thread
    for (int c0 = threadIdx.x; c0 < ch_hi; c0 += U * COMB_THREADS) {
        float4a v[U];
        // no branch around the reads (the compiler would wait for each one before the next):
        // chunks past the end re-read the last one and are not stored
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = lds4[min(c0 + u * COMB_THREADS, ch_hi - 1)];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int ch = c0 + u * COMB_THREADS;
            if (ch >= ch_lo && ch < ch_hi) I6_ROW_STORE(v[u], (float4a*)(base + 4 * ch));
        }
    }
    if (threadIdx.x < 8) {
        const int i = threadIdx.x < 4 ? 4 * (ch_lo - 1) + threadIdx.x : 4 * ch_hi + threadIdx.x - 4;
        if (i >= a && i < a + F && (i < 4 * ch_lo || i >= 4 * ch_hi)) base[i] = image[i];
    }
}

// chunks [c0, c1) of the line-aligned view of a row (base + 4 * chunk); chunk ch sits at lds4[ch - cofs]
__device__ inline void stream_tile(float* base, const int c0, const int c1, const int cofs, const float4a* lds4) {
    constexpr int U = 4;
    for (int ch0 = c0 + threadIdx.x; ch0 < c1; ch0 += U * COMB_THREADS) {
        float4a v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = lds4[min(ch0 + u * COMB_THREADS, c1 - 1) - cofs];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int ch = ch0 + u * COMB_THREADS;
            if (ch < c1) I6_ROW_STORE(v[u], (float4a*)(base + 4 * ch));
        }
    }
}

__device__ __forceinline__ float block_min256(float v, float* red) {
    v = wave_min_dpp(v);
    if ((threadIdx.x & 63) == 63) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
}
__device__ __forceinline__ float block_sum256(float v, float* red) {
    v = wave_sum_dpp(v);
    if ((threadIdx.x & 63) == 63) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// Sum of xs[c0, c1), every lane with a range of its own; called by whole waves.  Ranges of up to
// LONG_SLOT entries are summed by their lane.  Longer ones (the blank label of a CTC automaton,
// silence: one emission class on a large share of the edges) would keep one lane busy for
// microseconds per frame while the rest of the workgroup waits: the wave sums them together, 64
// entries at a time, in a fixed order.
constexpr int LONG_SLOT = 16;
__device__ __forceinline__ float slot_sum(const float* xs, const int c0, const int c1) {
    const int lane = threadIdx.x & 63;
    const bool is_long = c1 - c0 > LONG_SLOT;
    float s = 0.f;
    if (!is_long)
        for (int i = c0; i < c1; i++) s += xs[i];
    unsigned long long todo = __ballot(is_long);
    while (todo) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const int b0 = __builtin_amdgcn_readlane(c0, src), b1 = __builtin_amdgcn_readlane(c1, src);
        float p = 0.f;
        for (int q = b0 + lane; q < b1; q += 64) p += xs[q];
        p = lane63(wave_sum_dpp(p));
        if (lane == src) s = p;
    }
    return s;
}

// The same for MF frames whose staged values lie `stride` apart: the frames' LDS reads are independent of each other, so
// a lane's short range costs one read latency per entry for all of them.  Frame by frame the additions are slot_sum's.
template <int MF>
__device__ __forceinline__ void slot_sum_frames(const float* xs, const int stride, const int c0, const int c1, float (&s)[MF]) {
    const int lane = threadIdx.x & 63;
    const bool is_long = c1 - c0 > LONG_SLOT;
#pragma unroll
    for (int f = 0; f < MF; f++) s[f] = 0.f;
    if (!is_long)
        for (int i = c0; i < c1; i++) {
#pragma unroll
            for (int f = 0; f < MF; f++) s[f] += xs[f * stride + i];
        }
    unsigned long long todo = __ballot(is_long);
    while (todo) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const int b0 = __builtin_amdgcn_readlane(c0, src), b1 = __builtin_amdgcn_readlane(c1, src);
#pragma unroll
        for (int f = 0; f < MF; f++) {
            float p = 0.f;
            for (int q = b0 + lane; q < b1; q += 64) p += xs[f * stride + q];
            p = lane63(wave_sum_dpp(p));
            if (lane == src) s[f] = p;
        }
    }
}

// The same in log space, for the -log output (NEGLOG instances of the kernels below): xs holds the raw
// scores, +inf for a dead edge; the result is the smallest score m of the range and the sum of the
// 2^(m - x) over it -- {+inf, 0} if no edge of the range is alive.  The reference adds a slot's edges in
// log space too (fbw_op.cu:39-59,137-153) and so has a finite -log wherever some edge is alive, however
// small its share of the frame; sums of probabilities relative to the frame minimum flush to zero from
// 2^-126 of it and lose terms long before.
struct LogSum { float mn, sum; };
__device__ __forceinline__ LogSum slot_logsum(const float* xs, const int c0, const int c1) {
    const int lane = threadIdx.x & 63;
    const bool is_long = c1 - c0 > LONG_SLOT;
    LogSum r = { INF_F, 0.f };
    if (!is_long) {
        for (int i = c0; i < c1; i++) r.mn = fminf(r.mn, xs[i]);
        if (r.mn < INF_F)
            for (int i = c0; i < c1; i++) r.sum += __builtin_amdgcn_exp2f(r.mn - xs[i]);
    }
    unsigned long long todo = __ballot(is_long);
    while (todo) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const int b0 = __builtin_amdgcn_readlane(c0, src), b1 = __builtin_amdgcn_readlane(c1, src);
        float pm = INF_F;
        for (int q = b0 + lane; q < b1; q += 64) pm = fminf(pm, xs[q]);
        pm = lane63(wave_min_dpp(pm));
        float p = 0.f;
        if (pm < INF_F)
            for (int q = b0 + lane; q < b1; q += 64) p += __builtin_amdgcn_exp2f(pm - xs[q]);
        p = lane63(wave_sum_dpp(p));
        if (lane == src) { r.mn = pm; r.sum = p; }
    }
    return r;
}
// slot_logsum for MF frames whose staged scores lie `stride` apart (see slot_sum_frames); frame by frame slot_logsum's arithmetic
template <int MF>
__device__ __forceinline__ void slot_logsum_frames(const float* xs, const int stride, const int c0, const int c1, LogSum (&r)[MF]) {
    const int lane = threadIdx.x & 63;
    const bool is_long = c1 - c0 > LONG_SLOT;
#pragma unroll
    for (int f = 0; f < MF; f++) { r[f].mn = INF_F; r[f].sum = 0.f; }
    if (!is_long) {
        for (int i = c0; i < c1; i++) {
#pragma unroll
            for (int f = 0; f < MF; f++) r[f].mn = fminf(r[f].mn, xs[f * stride + i]);
        }
        for (int i = c0; i < c1; i++) {
#pragma unroll
            for (int f = 0; f < MF; f++)
                if (r[f].mn < INF_F) r[f].sum += __builtin_amdgcn_exp2f(r[f].mn - xs[f * stride + i]);
        }
    }
    unsigned long long todo = __ballot(is_long);
    while (todo) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const int b0 = __builtin_amdgcn_readlane(c0, src), b1 = __builtin_amdgcn_readlane(c1, src);
#pragma unroll
        for (int f = 0; f < MF; f++) {
            float pm = INF_F;
            for (int q = b0 + lane; q < b1; q += 64) pm = fminf(pm, xs[f * stride + q]);
            pm = lane63(wave_min_dpp(pm));
            float p = 0.f;
            if (pm < INF_F)
                for (int q = b0 + lane; q < b1; q += 64) p += __builtin_amdgcn_exp2f(pm - xs[f * stride + q]);
            p = lane63(wave_sum_dpp(p));
            if (lane == src) { r[f].mn = pm; r[f].sum = p; }
        }
    }
}
// a (+)= b for two pieces of one slot (edges staged in passes).  A slot that lies in one piece keeps the
// bits of that piece.
__device__ __forceinline__ void logsum_merge(LogSum& a, const LogSum b) {
    if (!(b.mn < INF_F)) return;
    if (!(a.mn < INF_F)) { a = b; return; }
    const float m = fminf(a.mn, b.mn);
    a.sum = a.sum * __builtin_amdgcn_exp2f(m - a.mn) + b.sum * __builtin_amdgcn_exp2f(m - b.mn);
    a.mn = m;
}
// Element of the -log output from a slot's log-space sum {m, s}, the frame minimum mn and log2 of the frame
// total (the sum of the 2^(mn - x) over all edges of the frame): -ln of s * 2^(mn - m) / total.
__device__ __forceinline__ float neg_log_value(const LogSum s, const float mn, const float logtot) {
    return s.mn < INF_F ? (((s.mn - mn) - __builtin_amdgcn_logf(s.sum)) + logtot) * LN2 : INF_F;
}

// (three waves per SIMD: with the headline workload's 48 KB row image three workgroups share a
// compute unit, and the register count must not stand in the way)
// NEGLOG: the instance for the -log output (I6FBW_OUT_NEG_LOG), which sums a slot's edges in log space.
// (At three waves per SIMD the -log instance keeps a few values of its paths for sequences of more than 1024 edges
// in scratch memory -- six reloads per frame there, none on the path for smaller sequences; at two it needs none, and
// the monophone configuration, all of whose sequences are small, takes 8 % longer per call.)
// SMALL: the instance for the sequences whose edges and slots stay in a thread's registers over a strip (comb_small: up
// to 1024 edges and 512 distinct emissions) and nothing else.  It needs a third of the registers, so that COMB_SMALL_OCC
// workgroups share a compute unit instead of three: a strip is a chain of dependent round trips (operands of a frame,
// block minimum, staging area, per-emission sums, block sum, row image, row out), and what hides them is the number of
// strips in flight -- with short rows (the row writer's domain: F below 2048 or a small tensor) the strips of a whole
// batch then run at the same time (monophone configuration: dense write 58 -> 42 us, call 0.194 -> 0.178 ms; four or six
// workgroups per unit measure the same, eight need 64 registers and spill: 50 us).  The host launches it next to the
// general instance, which leaves those sequences out (small_elsewhere).
// (with short rows -- batch: the launch has the LDS for several row images and a staging area of 2048 values -- also up to
// 2048 edges: a single pass through the staging area and two slots per thread where the general instance takes passes of
// 1024 edges with eight slots per thread and fetches sixteen edges per thread whatever their number)
__device__ __forceinline__ bool comb_small(const SeqMeta& m, const int batch) {
    return seq_error(m) == 0 && m.n_edges > 0 && m.L > 0 && m.n_edges <= (batch ? COMB_BATCH * COMB_BATCH_EDGES : COMB_XS) && m.D <= 2 * COMB_THREADS;
}
#ifndef I6_COMB_SMALL_OCC
#define I6_COMB_SMALL_OCC 6
#endif
constexpr int COMB_SMALL_OCC = I6_COMB_SMALL_OCC;
template <bool SYNC, bool NEGLOG, bool SMALL = false>
__global__ __launch_bounds__(COMB_THREADS, SMALL ? COMB_SMALL_OCC : 3) void fbw_combine(CombArgs a) {
    extern __shared__ float4a lds4[];
    __shared__ float redmin[COMB_THREADS / 64];
    __shared__ float redsum[COMB_THREADS / 64];
    static_assert(COMB_THREADS == 256, "block reductions assume 4 waves");

    // within a block of sequences the sequence index runs fastest: workgroups that run together
    // write neighbouring rows
    const int tid = threadIdx.x;
    int b, y;
    strip_index(a.B, &b, &y);
    const SeqMeta m = a.meta[b];
    if (!SMALL && a.pad_rows) {
        // Stage after stage there is nothing for fbw_padfill to run beside: its rows -- frames >= seq_len, for
        // this workgroup those among the eight frames at its own position in the sequence -- are written here,
        // one launch less in front of the recursion.
        const float hole = NEGLOG ? INF_F : 0.f;
        for (int t = max(y * TC, m.L); t < min(a.T, y * TC + TC); t++) {
            stream_const_row(a.out + t * a.ost_t + b * a.ost_b, a.F, hole);
            if (tid == 0) a.sum_output[(size_t)t * a.B + b] = 0.f;
        }
    }
    if (m.L == 0) return;                                      // rows of frames >= seq_len: above, or by fbw_padfill
    if (a.direct_only && !flat_direct(m)) return;
    if (SMALL ? !comb_small(m, a.batch_frames) : (a.small_elsewhere && comb_small(m, a.batch_frames))) return;
    const int T = a.T, B = a.B, F = a.F;
    // strips of TC frames are handed out from the middle of the sequence outwards: that is where the
    // forward and the backward recursion meet, so those rows are complete first
    const int n = (m.L + TC - 1) / TC;
    if (y >= n) return;
    const int strip = (y & 1) ? n / 2 - 1 - (y >> 1) : n / 2 + (y >> 1);
    const int t0 = strip * TC;
    const int tv = min(m.L, t0 + TC);    // frames [t0, tv) of this strip, all of them below seq_len
#ifdef I6_TRACE
    if (tid == 0) { atomicMin(&g_trace[2], wall_clock64()); if (b == 0) g_trace[1024 + strip] = wall_clock64(); }
#endif
    if (!SMALL && (seq_error(m) < 0 || m.n_edges == 0)) {
        // no recursion ran for this sequence: NaN for a reported problem, empty frames otherwise
        const bool err = seq_error(m) != 0;
        const float v = err ? __builtin_nanf("") : (a.out_mode != I6FBW_OUT_NEG_LOG ? 0.f : INF_F);
        for (int t = t0; t < tv; t++) {
            stream_const_row(a.out + t * a.ost_t + b * a.ost_b, a.F, v);
            if (tid == 0) a.sum_output[(size_t)t * a.B + b] = err ? __builtin_nanf("") : 0.f;
        }
        return;
    }
    if (SYNC) {
        // alpha rows [0, count_a) and beta rows [L - count_b, L) have been written through
        __shared__ int s_ok;
        if (tid == 0) {
            const int* prog = a.sync + SYNC_HDR + 2 * b;
            // the gather strips of these frames, then both recursions
            bool ok = true;
            const int* gflag = a.sync + SYNC_HDR + 2 * a.B + (size_t)b * ((a.T + TG - 1) / TG);
            const bool general = seq_error(m) > 0;      // no gather for it, and a recursion that takes its time
            for (int g = t0 / TG; !general && ok && g <= (tv - 1) / TG; g++) ok = spin_until_ge(gflag + g, 1, a.sync);
            for (int rep = 0; rep < (general ? 64 : 1); rep++) {
                ok = spin_until_ge(prog, tv, a.sync, general && rep < 63) && spin_until_ge(prog + 1, m.L - t0, a.sync, general && rep < 63);
                if (ok || load_agent(a.sync)) break;
            }
            s_ok = ok;
        }
        __syncthreads();
        if (!s_ok) {
            // timed out (reported through the abort flag): the rows say so too
            for (int t = t0; t < tv; t++) {
                stream_const_row(a.out + t * a.ost_t + b * a.ost_b, a.F, __builtin_nanf(""));
                if (tid == 0) a.sum_output[(size_t)t * a.B + b] = __builtin_nanf("");
            }
            return;
        }
    }
    if (!SMALL && seq_error(m) > 0) {
        __shared__ float gred[32];
        const long long soff = state_off(m.edge_begin, b);
        generic_combine<SYNC>(a.gen, m, b, t0, tv, T, B, F, a.out_mode, a.alpha + (size_t)T * soff, a.beta + (size_t)T * soff,
                              a.offA + (size_t)b * T, a.offB + (size_t)b * T, a.out, a.ost_t, a.ost_b, a.sum_output, gred);
        return;
    }
    constexpr bool prob = !NEGLOG;
    const float hole = prob ? 0.f : INF_F;
    const float psign = a.out_mode == I6FBW_OUT_NEG_PROB ? -1.f : 1.f;

    float* image = (float*)lds4;
    // the image is shifted by the row's offset within its 128-byte line; rows too long for LDS go
    // through it in tiles of tile_w floats
    const int F4 = a.tile_w ? a.tile_w >> 2 : (F + 32 + 3) >> 2;
    float* xs = image + 4 * F4;
    for (int i = tid; i < F4; i += COMB_THREADS) lds4[i] = (float4a){hole, hole, hole, hole};
    int a_prev = -1;                      // image shift of the previous frame

    const int nE = m.n_edges, D = m.D, SP = m.SP, DP = m.DP;
    const long long soff = state_off(m.edge_begin, b), goff = slot_off(m.edge_begin, b);
    const uint4* crec = a.crec + m.edge_begin;
    const int* cb = a.cbegin + goff;
    const int* de = a.demis + goff;
    const double* offA = a.offA + (size_t)b * T;
    const double* offB = a.offB + (size_t)b * T;
    const float* abase = a.alpha + (size_t)T * soff;
    const float* bbase = a.beta + (size_t)T * soff;
    const float* gbase = a.gtab + (size_t)T * goff;

    // writes the image positions of one frame from the per-slot sums (sd: sums of probabilities relative to
    // the frame minimum; NEGLOG: ls, the sums in log space), then streams the row out
    auto finish_row = [&](int t, float mn, float tot, const float* sd, const LogSum* ls, const int* em, int nslot_regs, double offs) {
        const bool dead = mn == INF_F;
        const float logtot = __builtin_amdgcn_logf(tot);
        if (tid == 0)
            a.sum_output[(size_t)t * B + b] = dead ? 0.f : (float)(((double)(mn - logtot) + offs) * (double)LN2);
        const float inv = dead ? 0.f : psign / tot;
        float* orow = a.out + t * a.ost_t + b * a.ost_b;
        const int sh = row_misalign(orow);
        if (!SMALL && a.tile_w) {
            // Row longer than the image: tile after tile of the line-aligned view of the row (positions
            // sh .. sh+F-1 of base = orow - sh).  The slots are ordered by emission index, but every
            // thread simply looks which of its slots fall into the tile; after the tile has gone out
            // their positions get the hole value back.
            auto value = [&](int js) -> float {
                if (prob) return sd[js] * inv;
                return dead ? INF_F : neg_log_value(ls[js], mn, logtot);
            };
            float* base = orow - sh;
            const int W = a.tile_w, P = sh + F;
            const int ch_lo = (sh + 3) >> 2, ch_hi = P >> 2;             // chunks that lie completely inside the row
            for (int p0 = 0; p0 < P; p0 += W) {
                const int p1 = min(p0 + W, P);
                for (int js = 0; js < nslot_regs; js++) {
                    const int p = sh + em[js];
                    if (tid + js * COMB_THREADS < D && p >= p0 && p < p1) image[p - p0] = value(js);
                }
                __syncthreads();
                stream_tile(base, max(p0 >> 2, ch_lo), min((p0 + W) >> 2, ch_hi), p0 >> 2, lds4);
                if (tid < 8) {                                            // the floats of the two cut chunks of the row
                    const int i = tid < 4 ? 4 * (ch_lo - 1) + tid : 4 * ch_hi + tid - 4;
                    if (i >= sh && i < P && (i < 4 * ch_lo || i >= 4 * ch_hi) && i >= p0 && i < p1) base[i] = image[i - p0];
                }
                __syncthreads();
                for (int js = 0; js < nslot_regs; js++) {
                    const int p = sh + em[js];
                    if (tid + js * COMB_THREADS < D && p >= p0 && p < p1) image[p - p0] = hole;
                }
                __syncthreads();
            }
            return;
        }
        if (a_prev >= 0 && a_prev != sh) {
            for (int js = 0; js < nslot_regs; js++)
                if (tid + js * COMB_THREADS < D) image[a_prev + em[js]] = hole;
            __syncthreads();
        }
        a_prev = sh;
        for (int js = 0; js < nslot_regs; js++) {
            const int d = tid + js * COMB_THREADS;
            if (d < D) {
                float v;
                if (prob) v = sd[js] * inv;
                else v = dead ? INF_F : neg_log_value(ls[js], mn, logtot);
                image[sh + em[js]] = v;
            }
        }
        __syncthreads();
        stream_image_row(orow, F, lds4, image);
    };

    // Small sequences, short rows: several frames at a time.  Every step of a frame -- minimum, staging, per-emission
    // sums, total, row image, row -- is an LDS round trip and a barrier for four waves, about 400 cycles each whatever
    // the amount of work, and a frame has ten of them (1.8 us per frame for 30 edges as for 400); taken for MF frames
    // together they cost the same once.  Four frames with two edges per thread, two with four or one with eight, in the same
    // registers and the same LDS.  Same arithmetic in the same order as the path below, frame by frame, hence the same
    // bits, in the -log instance too.  (50 x 2 x 10: 0.052 -> 0.047 ms per call; 500 x 32 x 264: row writer 44 -> 38 us.)
    __shared__ float red4[2][COMB_BATCH][COMB_THREADS / 64];
    auto batched = [&](auto mf_, auto je_) {
        constexpr int MF = decltype(mf_)::value, JE = decltype(je_)::value, JS = 2, XSTRIDE = JE * COMB_THREADS;
        static_assert(MF <= COMB_BATCH && MF * XSTRIDE <= COMB_BATCH * COMB_BATCH_EDGES, "LDS of the launch: comb_batch_lds_bytes");
        float* xsb = image + (size_t)MF * 4 * F4;                 // MF x XSTRIDE staged values
        for (int i = F4 + tid; i < MF * F4; i += COMB_THREADS) lds4[i] = (float4a){hole, hole, hole, hole};      // (the first image: above)
        unsigned eft[JE], esl[JE];           // source | target << 16, slot
        float ew[JE];
#pragma unroll
        for (int j = 0; j < JE; j++) {
            const int i = tid + j * COMB_THREADS;
            uint4 r = make_uint4(0u, __float_as_uint(INF_F), 0u, 0u);     // weight +inf: contributes nothing
            if (i < nE) r = crec[i];
            eft[j] = r.x; esl[j] = r.z; ew[j] = __uint_as_float(r.y);
        }
        int c0[JS], c1[JS], em[JS];
#pragma unroll
        for (int js = 0; js < JS; js++) {
            const int d = tid + js * COMB_THREADS;
            c0[js] = c1[js] = em[js] = 0;
            if (d < D) { c0[js] = cb[d]; c1[js] = cb[d + 1]; em[js] = de[d]; }
        }
        const int wave = tid >> 6, lane = tid & 63;
        for (int tb = t0; tb < tv; tb += MF) {
            const int nf = min(MF, tv - tb);
            // operands of all frames of the batch in one round trip (frames past the end: the last one once more, unused)
            float x[MF][JE], lmin[MF];
            // the row offsets: lane 2f has the alpha row's of frame f, lane 2f+1 the beta row's
            const double voff = tid < 2 * nf ? load_x<SYNC>(((tid & 1) ? offB : offA) + tb + (tid >> 1)) : 0.0;
            {
                float va[MF][JE], vb[MF][JE], vg[MF][JE];
#pragma unroll
                for (int f = 0; f < MF; f++) {
                    const int t = min(tb + f, tv - 1);
                    const float* arow = abase + (size_t)t * SP;
                    const float* brow = bbase + (size_t)t * SP;
                    const float* grow = gbase + (size_t)t * DP;
#pragma unroll
                    for (int j = 0; j < JE; j++) {
                        va[f][j] = load_x<SYNC>(arow + (eft[j] & 0xFFFFu)); vb[f][j] = load_x<SYNC>(brow + (eft[j] >> 16)); vg[f][j] = load_x<SYNC>(grow + esl[j]);
                    }
                }
#pragma unroll
                for (int f = 0; f < MF; f++) {
                    lmin[f] = INF_F;
#pragma unroll
                    for (int j = 0; j < JE; j++) { x[f][j] = (va[f][j] + ew[j]) + (vg[f][j] + vb[f][j]); lmin[f] = fminf(lmin[f], x[f][j]); }
                }
            }
            float mn[MF];
#pragma unroll
            for (int f = 0; f < MF; f++) {
                const float v = wave_min_dpp(lmin[f]);
                if (lane == 63) red4[0][f][wave] = v;
            }
            __syncthreads();
            // staged per frame: the probabilities relative to the frame minimum (-log instance: the raw scores, and
            // the frame normaliser is the sum over the edges, in edge order per thread, as in the path below)
            float part[MF];
#pragma unroll
            for (int f = 0; f < MF; f++) {
                mn[f] = fminf(fminf(red4[0][f][0], red4[0][f][1]), fminf(red4[0][f][2], red4[0][f][3]));
                part[f] = 0.f;
#pragma unroll
                for (int j = 0; j < JE; j++) {
                    const float p = mn[f] == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn[f] - x[f][j]);
                    if (NEGLOG) part[f] += p;
                    xsb[f * XSTRIDE + tid + j * COMB_THREADS] = NEGLOG ? x[f][j] : p;
                }
            }
            // per-emission sums in fixed (input) order and the frame normalisers
            float val[MF][JS], tot[MF];
            if (!NEGLOG) {
                __syncthreads();
#pragma unroll
                for (int js = 0; js < JS; js++) {
                    float s4[MF];
                    slot_sum_frames<MF>(xsb, XSTRIDE, c0[js], c1[js], s4);
#pragma unroll
                    for (int f = 0; f < MF; f++) val[f][js] = s4[f];
                }
#pragma unroll
                for (int f = 0; f < MF; f++)
#pragma unroll
                    for (int js = 0; js < JS; js++) part[f] += val[f][js];
            }
#pragma unroll
            for (int f = 0; f < MF; f++) {
                const float v = wave_sum_dpp(part[f]);
                if (lane == 63) red4[1][f][wave] = v;
            }
            __syncthreads();              // (-log instance: also publishes the staged scores)
#pragma unroll
            for (int f = 0; f < MF; f++) tot[f] = (red4[1][f][0] + red4[1][f][1]) + (red4[1][f][2] + red4[1][f][3]);
            if (NEGLOG) {
#pragma unroll
                for (int js = 0; js < JS; js++) {
                    LogSum l4[MF];
                    slot_logsum_frames<MF>(xsb, XSTRIDE, c0[js], c1[js], l4);
#pragma unroll
                    for (int f = 0; f < MF; f++)
                        val[f][js] = mn[f] == INF_F ? INF_F : neg_log_value(l4[f], mn[f], __builtin_amdgcn_logf(tot[f]));
                }
            }
            // loss, image positions, rows
            int shf[MF];
#pragma unroll
            for (int f = 0; f < MF; f++) {
                const double offs = __shfl(voff, 2 * f) + __shfl(voff, 2 * f + 1);
                shf[f] = 0;
                if (f < nf) {
                    const int t = tb + f;
                    const bool dead = mn[f] == INF_F;
                    const float logtot = __builtin_amdgcn_logf(tot[f]);
                    if (tid == 0) a.sum_output[(size_t)t * B + b] = dead ? 0.f : (float)(((double)(mn[f] - logtot) + offs) * (double)LN2);
                    const float inv = dead ? 0.f : psign / tot[f];
                    shf[f] = row_misalign(a.out + t * a.ost_t + b * a.ost_b);
#pragma unroll
                    for (int js = 0; js < JS; js++)
                        if (tid + js * COMB_THREADS < D) image[(size_t)f * 4 * F4 + shf[f] + em[js]] = NEGLOG ? val[f][js] : val[f][js] * inv;
                }
            }
            __syncthreads();
#pragma unroll
            for (int f = 0; f < MF; f++)
                if (f < nf) stream_image_row(a.out + (tb + f) * a.ost_t + b * a.ost_b, F, lds4 + (size_t)f * F4, image + (size_t)f * 4 * F4);
            __syncthreads();
#pragma unroll
            for (int f = 0; f < MF; f++)
                if (f < nf) {
#pragma unroll
                    for (int js = 0; js < JS; js++)
                        if (tid + js * COMB_THREADS < D) image[(size_t)f * 4 * F4 + shf[f] + em[js]] = hole;
                }
        }
    };
    bool written = false;
    if constexpr (SMALL) {
        if (a.batch_frames && nE <= COMB_BATCH_EDGES) {
            batched(std::integral_constant<int, COMB_BATCH>{}, std::integral_constant<int, COMB_BATCH_EDGES / COMB_THREADS>{});
            written = true;
        } else if (a.batch_frames && nE <= COMB_XS) {
            batched(std::integral_constant<int, COMB_BATCH / 2>{}, std::integral_constant<int, COMB_XS / COMB_THREADS>{});
            written = true;
        } else if (a.batch_frames) {
            batched(std::integral_constant<int, 1>{}, std::integral_constant<int, COMB_BATCH * COMB_BATCH_EDGES / COMB_THREADS>{});
            written = true;
        }
    }
    if (written) {
    } else if (SMALL || (nE <= COMB_XS && D <= 2 * COMB_THREADS)) {
        // fast path: this thread's edges and slots stay in registers for the whole strip, and
        // the operands of the next frame are fetched while the current one is processed
        constexpr int JE = COMB_XS / COMB_THREADS, JS = 2;
        unsigned efr[JE], eto[JE], esl[JE];
        float ew[JE];
#pragma unroll
        for (int j = 0; j < JE; j++) {
            const int i = tid + j * COMB_THREADS;
            uint4 r = make_uint4(0u, __float_as_uint(INF_F), 0u, 0u);     // weight +inf: contributes nothing
            if (i < nE) r = crec[i];
            efr[j] = r.x & 0xFFFFu; eto[j] = r.x >> 16; esl[j] = r.z; ew[j] = __uint_as_float(r.y);
        }
        int c0[JS], c1[JS], em[JS];
#pragma unroll
        for (int js = 0; js < JS; js++) {
            const int d = tid + js * COMB_THREADS;
            c0[js] = c1[js] = em[js] = 0;
            if (d < D) { c0[js] = cb[d]; c1[js] = cb[d + 1]; em[js] = de[d]; }
        }
        float va[JE], vb[JE], vg[JE];
        double voff = 0.0;
        auto fetch = [&](int t) {
            const float* arow = abase + (size_t)t * SP;
            const float* brow = bbase + (size_t)t * SP;
            const float* grow = gbase + (size_t)t * DP;
#pragma unroll
            for (int j = 0; j < JE; j++) {
                va[j] = load_x<SYNC>(arow + efr[j]); vb[j] = load_x<SYNC>(brow + eto[j]); vg[j] = load_x<SYNC>(grow + esl[j]);
            }
            if (tid == 0) voff = load_x<SYNC>(offA + t) + load_x<SYNC>(offB + t);
        };
        fetch(t0);
        for (int t = t0; t < tv; t++) {
            // edge scores x = alpha_t[from] + w + am + beta_{t+1}[to]   (fbw_op.cu:93-100)
            float x[JE];
            float lmin = INF_F;
#pragma unroll
            for (int j = 0; j < JE; j++) { x[j] = (va[j] + ew[j]) + (vg[j] + vb[j]); lmin = fminf(lmin, x[j]); }
            const double offs = voff;
            if (t + 1 < tv) fetch(t + 1);
            const float mn = block_min256(lmin, redmin);
            // The frame normaliser (fbw_op.cu:115-134) is the sum of the probabilities relative to the frame
            // minimum: of the per-emission sums, or, in the -log instance, which has no such sums, of the edges'
            // in edge order per thread -- on every path of either dense writer edge i belongs to thread i mod 256,
            // so each instance gives the same bits wherever it runs.
            float part = 0.f;
#pragma unroll
            for (int j = 0; j < JE; j++) {
                const float p = mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - x[j]);
                if (NEGLOG) part += p;
                xs[tid + j * COMB_THREADS] = NEGLOG ? x[j] : p;
            }
            float tot = 0.f;
            if (NEGLOG) tot = block_sum256(part, redsum);     // (its barrier also publishes xs)
            else __syncthreads();
            // per-emission sums in fixed (input) order
            float sd[JS];
            LogSum ls[JS];
#pragma unroll
            for (int js = 0; js < JS; js++) {
                if (NEGLOG) ls[js] = slot_logsum(xs, c0[js], c1[js]);
                else { sd[js] = slot_sum(xs, c0[js], c1[js]); part += sd[js]; }
            }
            if (!NEGLOG) tot = block_sum256(part, redsum);
            finish_row(t, mn, tot, sd, ls, em, JS, offs);
        }
    } else if (!SMALL && nE <= COMB_MID_EDGES && D <= COMB_MID_SLOTS) {
        // medium sequences: this thread's edges still stay in registers for the whole strip (sixteen
        // of them, source and target packed), the operands of a frame are fetched in one go, and the
        // scores go through the LDS staging area in up to four passes
        constexpr int JE = COMB_MID_EDGES / COMB_THREADS, JS = COMB_MID_SLOTS / COMB_THREADS, JP = COMB_XS / COMB_THREADS;
        unsigned eft[JE], esl[JE];
        float ew[JE];
#pragma unroll
        for (int j = 0; j < JE; j++) {
            const int i = tid + j * COMB_THREADS;
            uint4 r = make_uint4(0u, __float_as_uint(INF_F), 0u, 0u);     // weight +inf: contributes nothing
            if (i < nE) r = crec[i];
            eft[j] = r.x; esl[j] = r.z; ew[j] = __uint_as_float(r.y);
        }
        int em[JS];
#pragma unroll
        for (int js = 0; js < JS; js++) {
            const int d = tid + js * COMB_THREADS;
            em[js] = d < D ? de[d] : 0;
        }
        const int npass = (nE + COMB_XS - 1) / COMB_XS;
        for (int t = t0; t < tv; t++) {
            const float* arow = abase + (size_t)t * SP;
            const float* brow = bbase + (size_t)t * SP;
            const float* grow = gbase + (size_t)t * DP;
            float x[JE];
            float lmin = INF_F;
#pragma unroll
            for (int j = 0; j < JE; j++) {
                x[j] = (load_x<SYNC>(arow + (eft[j] & 0xFFFFu)) + ew[j]) + (load_x<SYNC>(grow + esl[j]) + load_x<SYNC>(brow + (eft[j] >> 16)));
                lmin = fminf(lmin, x[j]);
            }
            const double offs = tid == 0 ? load_x<SYNC>(offA + t) + load_x<SYNC>(offB + t) : 0.0;
            const float mn = block_min256(lmin, redmin);
            float sd[JS];
            LogSum ls[JS];
#pragma unroll
            for (int js = 0; js < JS; js++) { sd[js] = 0.f; ls[js].mn = INF_F; ls[js].sum = 0.f; }
            float part = 0.f;         // see the fast path
#pragma unroll
            for (int p = 0; p < JE / JP; p++) {
                if (p < npass) {
                    const int p0 = p * COMB_XS, p1 = min(nE, p0 + COMB_XS);
                    if (p > 0) __syncthreads();
#pragma unroll
                    for (int jj = 0; jj < JP; jj++) {
                        const float pr = mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - x[p * JP + jj]);
                        if (NEGLOG) part += pr;
                        xs[tid + jj * COMB_THREADS] = NEGLOG ? x[p * JP + jj] : pr;
                    }
                    __syncthreads();
#pragma unroll
                    for (int js = 0; js < JS; js++) {
                        const int d = tid + js * COMB_THREADS;
                        int e0 = 0, e1 = 0;
                        if (d < D) { e0 = max(cb[d], p0) - p0; e1 = min(cb[d + 1], p1) - p0; }
                        if (NEGLOG) logsum_merge(ls[js], slot_logsum(xs, e0, e1));
                        else sd[js] += slot_sum(xs, e0, e1);
                    }
                }
            }
            if (!NEGLOG) {
#pragma unroll
                for (int js = 0; js < JS; js++) part += sd[js];
            }
            const float tot = block_sum256(part, redsum);
            finish_row(t, mn, tot, sd, ls, em, JS, offs);
        }
    } else if (!SMALL) {
        // general path: edge records re-read per frame, edges staged through LDS in passes of
        // COMB_XS, per-slot sums accumulated across the passes
        for (int t = t0; t < tv; t++) {
            const float* arow = abase + (size_t)t * SP;
            const float* brow = bbase + (size_t)t * SP;
            const float* grow = gbase + (size_t)t * DP;
            auto score = [&](int i) {
                const uint4 r = crec[i];
                return (load_x<SYNC>(arow + (r.x & 0xFFFFu)) + __uint_as_float(r.y)) + (load_x<SYNC>(grow + r.z) + load_x<SYNC>(brow + (r.x >> 16)));
            };
            float lmin = INF_F;
            for (int i = tid; i < nE; i += COMB_THREADS) lmin = fminf(lmin, score(i));
            const float mn = block_min256(lmin, redmin);
            float sd[COMB_JD];
            LogSum ls[COMB_JD];
            int em[COMB_JD];
#pragma unroll
            for (int jd = 0; jd < COMB_JD; jd++) { sd[jd] = 0.f; ls[jd].mn = INF_F; ls[jd].sum = 0.f; em[jd] = 0; }
            float part = 0.f;         // see the fast path
            for (int p0 = 0; p0 < nE; p0 += COMB_XS) {
                const int p1 = min(nE, p0 + COMB_XS);
                __syncthreads();
                for (int i = p0 + tid; i < p1; i += COMB_THREADS) {
                    const float x = score(i);
                    const float pr = mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - x);
                    if (NEGLOG) part += pr;
                    xs[i - p0] = NEGLOG ? x : pr;
                }
                __syncthreads();
#pragma unroll
                for (int jd = 0; jd < COMB_JD; jd++) {
                    const int d = tid + jd * COMB_THREADS;
                    int e0 = 0, e1 = 0;
                    if (d < D) { e0 = max(cb[d], p0) - p0; e1 = min(cb[d + 1], p1) - p0; }
                    if (NEGLOG) logsum_merge(ls[jd], slot_logsum(xs, e0, e1));
                    else sd[jd] += slot_sum(xs, e0, e1);
                }
            }
#pragma unroll
            for (int jd = 0; jd < COMB_JD; jd++) {
                const int d = tid + jd * COMB_THREADS;
                if (d < D) em[jd] = de[d];
                if (!NEGLOG) part += sd[jd];
            }
            const float tot = block_sum256(part, redsum);
            finish_row(t, mn, tot, sd, ls, em, COMB_JD, load_x<SYNC>(offA + t) + load_x<SYNC>(offB + t));
        }
    }
}

// ---------------------------------------------------------------------------------------------
// stage 4, flat form (fbw_flat).  The dense tensor is mostly holes: of the 12001 floats of a row of
// the headline workload about 370 carry a posterior.  Here the posteriors of a frame are first
// computed in compact form (one float per distinct emission of the sequence), and the tensor is
// then written as a flat sequence of 128-byte-aligned spans of FLAT_W floats, whatever the row
// length: a span is built in LDS from the (at most two) compact rows it cuts and leaves as two
// aligned 16-byte stores per thread.
//
// One kernel holds both kinds of job, in one dispatch order:
//   posterior job (sequence b, FLAT_TCF frames): waits for the two recursions to have passed its
//       frames, computes edge scores, frame normaliser and per-emission sums as fbw_combine does,
//       writes loss and compact posteriors and raises the flag of its frames;
//   write job (group, j): FLAT_KMAX spans of the group's rows; waits for the flags of the rows they
//       cut.  A group is a strip of TC frames of all sequences (layout (T,B,F)) or of one sequence
//       (layout (B,T,F)), i.e. a contiguous piece of the tensor, clipped to whole rows: lines cut
//       by the ends of a group are shared with the neighbouring group and written element by
//       element by both.
// Strips are taken from the middle outwards (where the recursions meet), posterior jobs FLAT_AHEAD
// strips ahead of the write jobs that need them.  Workgroups are dispatched in index order and a
// job only ever waits for jobs with a smaller index (and for the recursion, which is resident before
// this kernel starts), so the job that is waited for is running or done: no wait can block the
// kernel, whatever the occupancy.
//
// Measured on the headline tensor (1.54 GB): bare writers with jobs of this shape (8 strided spans, built
// in LDS, two 16-byte stores per thread) reach 5.6-5.9 TB/s whatever the occupancy, also as persistent
// workers; 6.9 TB/s needs a fresh workgroup per single span at two per compute unit, i.e. jobs with
// nothing to read.  This kernel writes the tensor in 0.265 ms when it has the machine to itself
// (5.8 TB/s; 0.30 ms for fbw_combine + fbw_padfill) and spends the same beside the recursion.  Its time
// does not change when the reads of the write jobs are taken out or when a workgroup waits for the
// stores of each span before the next: it is bound by the memory system's rate for these writes.
// ---------------------------------------------------------------------------------------------
constexpr int FLAT_W = 2048;                  // floats per span: two 16-byte stores per thread
#ifndef I6_FLAT_AHEAD
#define I6_FLAT_AHEAD 6
#endif
#ifndef I6_FLAT_AHEAD_ALONE
#define I6_FLAT_AHEAD_ALONE 4
#endif
#ifndef I6_FLAT_KMAX
#define I6_FLAT_KMAX 8
#endif
#ifndef I6_FLAT_OCC
#define I6_FLAT_OCC 8
#endif
// strips by which posterior jobs run ahead of the write jobs that need them: beside the recursion, whose
// progress the posterior jobs wait for (headline 0.513 ms with 4, 0.508 with 6, 0.515 with 8), and with
// everything ready when the kernel starts (config 4: dense write 0.193 ms with 4, 0.203 with 6)
constexpr int FLAT_AHEAD = I6_FLAT_AHEAD, FLAT_AHEAD_ALONE = I6_FLAT_AHEAD_ALONE;
constexpr int FLAT_KMAX = I6_FLAT_KMAX;       // spans per write job
constexpr int FLAT_MIN_F = FLAT_W;            // a span then cuts at most two rows
constexpr unsigned FLAT_SKIP = 0x7fc0deadu;   // image marker, a NaN no computation produces: element not written by this job

struct FlatArgs {
    CombArgs c;
    int layout;            // 0: out is (T, B, F) contiguous, 1: (B, T, F) contiguous
    int nW;                // write jobs per group
    int K;                 // spans per write job
    int ahead;             // strips by which posterior jobs are dispatched ahead of the write jobs that need them
    int shift;             // floats between the 128-byte line boundary below out and out
    int* cflag;            // per (sequence, strip): 1 compact posteriors written, 2 given up
    const int* wpfx; int wpfx_stride;
    float* cp;             // compact posteriors [seq][t][slot], in the memory of the compact emission table:
                           // row t of that table is last read by the posterior job that then overwrites it
};

// i-th strip of n in the order middle, middle+1, middle-1, middle+2, ... (the side that runs out first is skipped)
__device__ __forceinline__ int middle_out(const int i, const int n, const int mid) {
    const int up = n - 1 - mid, down = mid;
    if (i <= 2 * min(up, down)) return (i & 1) ? mid + (i + 1) / 2 : mid - i / 2;
    return up > down ? mid + (i - down) : mid - (i - up);
}

template <bool SYNC, bool NEGLOG>
__device__ __forceinline__ void flat_post(const FlatArgs& fa, const int b, const int t0, float* xs, float* redmin, float* redsum,
                                          int* s_ok) {
    const CombArgs& a = fa.c;
    const int tid = threadIdx.x;
    const SeqMeta m = a.meta[b];
    const int T = a.T, B = a.B;
    const int t1 = min(T, t0 + FLAT_TCF);
    if (t0 >= T) return;
    const int L = m.L;
    // frames from seq_len on: loss 0 (fbw_op.cu:120-128); their rows are holes, written by the write jobs
    for (int t = max(t0, L) + tid; t < t1; t += COMB_THREADS) a.sum_output[(size_t)t * B + b] = 0.f;
    const int tv = min(L, t1);
    if (t0 >= tv) return;
    const int err = seq_error(m);
    if (err < 0 || m.n_edges == 0) {
        for (int t = t0 + tid; t < tv; t += COMB_THREADS) a.sum_output[(size_t)t * B + b] = err < 0 ? __builtin_nanf("") : 0.f;
        return;
    }
    if (!flat_fast(m)) return;              // fbw_combine writes loss and rows of this sequence
    int* flag = fa.cflag + (size_t)b * ((T + FLAT_TCF - 1) / FLAT_TCF) + t0 / FLAT_TCF;
    if (SYNC) {
        if (tid == 0) {
            const int* prog = a.sync + SYNC_HDR + 2 * b;
            const int* gflag = a.sync + SYNC_HDR + 2 * a.B + (size_t)b * ((a.T + TG - 1) / TG);
            bool ok = true;
            for (int g = t0 / TG; ok && g <= (tv - 1) / TG; g++) ok = spin_until_ge(gflag + g, 1, a.sync);
            ok = ok && spin_until_ge(prog, tv, a.sync) && spin_until_ge(prog + 1, m.L - t0, a.sync);
            *s_ok = ok;
        }
        __syncthreads();
        if (!*s_ok) {
            for (int t = t0 + tid; t < tv; t += COMB_THREADS) a.sum_output[(size_t)t * B + b] = __builtin_nanf("");
            wait_stores();
            __syncthreads();
            if (tid == 0) store_agent(flag, 2);
            return;
        }
    }
    // (A run-time value in the instance for the posterior modes, although the host launches the NEGLOG instance for the
    // -log output: with the branch folded away the compiler arranges the rest so that it needs five registers more
    // than the 64 this kernel is launched for, and spills them inside the frame loop.)
    const bool prob = NEGLOG ? false : a.out_mode != I6FBW_OUT_NEG_LOG;
    const float psign = a.out_mode == I6FBW_OUT_NEG_PROB ? -1.f : 1.f;
    const int nE = m.n_edges, D = m.D, SP = m.SP, DP = m.DP;
    const long long soff = state_off(m.edge_begin, b), goff = slot_off(m.edge_begin, b);
    const uint4* crec = a.crec + m.edge_begin;
    const int* cb = a.cbegin + goff;
    const double* offA = a.offA + (size_t)b * T;
    const double* offB = a.offB + (size_t)b * T;
    const float* abase = a.alpha + (size_t)T * soff;
    const float* bbase = a.beta + (size_t)T * soff;
    const float* gbase = a.gtab + (size_t)T * goff;
    float* cpbase = fa.cp + (size_t)T * goff;

    constexpr int JE = COMB_FAST_EDGES / COMB_THREADS;
    if (nE > COMB_FAST_EDGES || D > COMB_FAST_SLOTS) {
        // Larger sequences: the edges of a frame in pieces of COMB_FAST_EDGES (records re-read from the
        // cache per frame), raw scores parked in the staging area until the frame minimum is known.
        constexpr int JSL = FLAT_SLOTS / COMB_THREADS;
        float* xs_all = xs;       // scores of all edges, frame by frame
        unsigned crl[JSL];
#pragma unroll
        for (int js = 0; js < JSL; js++) {
            const int d = tid + js * COMB_THREADS;
            crl[js] = d < D ? (unsigned)cb[d] | ((unsigned)cb[d + 1] << 16) : 0u;
        }
        // (a piece of the edge records serves all frames of the job: one round trip for the records, one for
        // the operands of all frames, per piece)
        const int nf = tv - t0;
        float lmins[FLAT_TCF];
        double voffs[FLAT_TCF];
#pragma unroll
        for (int f = 0; f < FLAT_TCF; f++) {
            lmins[f] = INF_F; voffs[f] = 0.0;
            if (tid == 0 && f < nf) voffs[f] = load_x<SYNC>(offA + t0 + f) + load_x<SYNC>(offB + t0 + f);
        }
        for (int c0 = 0; c0 < nE; c0 += COMB_FAST_EDGES) {
            uint4 r[JE];
            float va[FLAT_TCF][JE], vb[FLAT_TCF][JE], vg[FLAT_TCF][JE];
#pragma unroll
            for (int j = 0; j < JE; j++) {
                const int i = c0 + tid + j * COMB_THREADS;
                r[j] = make_uint4(0u, __float_as_uint(INF_F), 0u, 0u);     // weight +inf: contributes nothing
                if (i < nE) r[j] = crec[i];
            }
#pragma unroll
            for (int f = 0; f < FLAT_TCF; f++) {
                const int t = min(t0 + f, tv - 1);
                const float* arow = abase + (size_t)t * SP;
                const float* brow = bbase + (size_t)t * SP;
                const float* grow = gbase + (size_t)t * DP;
#pragma unroll
                for (int j = 0; j < JE; j++) {
                    va[f][j] = load_x<SYNC>(arow + (r[j].x & 0xFFFFu)); vb[f][j] = load_x<SYNC>(brow + (r[j].x >> 16)); vg[f][j] = load_x<SYNC>(grow + r[j].z);
                }
            }
#pragma unroll
            for (int f = 0; f < FLAT_TCF; f++) {
#pragma unroll
                for (int j = 0; j < JE; j++) {
                    const int i = c0 + tid + j * COMB_THREADS;
                    const float x = (va[f][j] + __uint_as_float(r[j].y)) + (vg[f][j] + vb[f][j]);     // same order as below
                    if (i < nE) xs_all[f * FLAT_EDGES + i] = x;
                    lmins[f] = fminf(lmins[f], x);
                }
            }
        }
#pragma unroll
        for (int f = 0; f < FLAT_TCF; f++) {
            if (f >= nf) break;
            const int t = t0 + f;
            float* xs = xs_all + f * FLAT_EDGES;
            const float lmin = lmins[f];
            const double offs = voffs[f];
            const float mn = block_min256(lmin, redmin);
            float sd[JSL];
            LogSum ls[JSL];
            float tot;
            if (NEGLOG) {
                float part = 0.f;         // the frame normaliser, as in fbw_combine
                for (int i = tid; i < nE; i += COMB_THREADS) part += mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - xs[i]);
                tot = block_sum256(part, redsum);
#pragma unroll
                for (int js = 0; js < JSL; js++) ls[js] = slot_logsum(xs, (int)(crl[js] & 0xFFFFu), (int)(crl[js] >> 16));
            } else {
                for (int i = tid; i < nE; i += COMB_THREADS) xs[i] = mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - xs[i]);    // (each thread its own)
                __syncthreads();
                float lsum = 0.f;
#pragma unroll
                for (int js = 0; js < JSL; js++) {
                    sd[js] = slot_sum(xs, (int)(crl[js] & 0xFFFFu), (int)(crl[js] >> 16));
                    lsum += sd[js];
                }
                tot = block_sum256(lsum, redsum);
            }
            const bool dead = mn == INF_F;
            const float logtot = __builtin_amdgcn_logf(tot);
            if (tid == 0)
                a.sum_output[(size_t)t * B + b] = dead ? 0.f : (float)(((double)(mn - logtot) + offs) * (double)LN2);
            const float inv = dead ? 0.f : psign / tot;
            float* cprow = cpbase + (size_t)t * DP;
#pragma unroll
            for (int js = 0; js < JSL; js++) {
                const int d = tid + js * COMB_THREADS;
                if (d < D) {
                    float v;
                    if (prob) v = sd[js] * inv;
                    else if (NEGLOG) v = dead ? INF_F : neg_log_value(ls[js], mn, logtot);
                    else v = (dead || sd[js] == 0.f) ? INF_F : (logtot - __builtin_amdgcn_logf(sd[js])) * LN2;
                    store_agent(cprow + d, v);
                }
            }
        }
        wait_stores();
        __syncthreads();
        if (tid == 0) store_agent(flag, 1);
        return;
    }
    // this thread's edges and slots stay in registers for the whole strip
    constexpr int JS = COMB_FAST_SLOTS / COMB_THREADS;
    unsigned eft[JE], esl[JE];
    float ew[JE];
#pragma unroll
    for (int j = 0; j < JE; j++) {
        const int i = tid + j * COMB_THREADS;
        uint4 r = make_uint4(0u, __float_as_uint(INF_F), 0u, 0u);     // weight +inf: contributes nothing
        if (i < nE) r = crec[i];
        eft[j] = r.x; esl[j] = r.z; ew[j] = __uint_as_float(r.y);
    }
    unsigned cr[JS];          // first edge | one past the last edge << 16 of my slots
#pragma unroll
    for (int js = 0; js < JS; js++) {
        const int d = tid + js * COMB_THREADS;
        cr[js] = d < D ? (unsigned)cb[d] | ((unsigned)cb[d + 1] << 16) : 0u;
    }
    // the operands of the next frame are fetched while the current one is processed
    float va[JE], vb[JE], vg[JE];
    double voff = 0.0;
    auto fetch = [&](int t) {
        const float* arow = abase + (size_t)t * SP;
        const float* brow = bbase + (size_t)t * SP;
        const float* grow = gbase + (size_t)t * DP;
#pragma unroll
        for (int j = 0; j < JE; j++) {
            va[j] = load_x<SYNC>(arow + (eft[j] & 0xFFFFu)); vb[j] = load_x<SYNC>(brow + (eft[j] >> 16)); vg[j] = load_x<SYNC>(grow + esl[j]);
        }
        if (tid == 0) voff = load_x<SYNC>(offA + t) + load_x<SYNC>(offB + t);
    };
    fetch(t0);
    for (int t = t0; t < tv; t++) {
        // edge scores x = alpha_t[from] + w + am + beta_{t+1}[to]   (fbw_op.cu:93-100)
        float x[JE];
        float lmin = INF_F;
#pragma unroll
        for (int j = 0; j < JE; j++) { x[j] = (va[j] + ew[j]) + (vg[j] + vb[j]); lmin = fminf(lmin, x[j]); }
        const double offs = voff;
        if (t + 1 < tv) fetch(t + 1);
        const float mn = block_min256(lmin, redmin);
        // the frame normaliser (fbw_op.cu:115-134), as in fbw_combine
        float sd[JS];
        LogSum ls[JS];
        float tot;
        if (NEGLOG) {
            float part = 0.f;
#pragma unroll
            for (int j = 0; j < JE; j++) {
                part += mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - x[j]);
                xs[tid + j * COMB_THREADS] = x[j];
            }
            tot = block_sum256(part, redsum);      // (its barrier also publishes xs)
            // per-emission sums in fixed (input) order
#pragma unroll
            for (int js = 0; js < JS; js++) ls[js] = slot_logsum(xs, (int)(cr[js] & 0xFFFFu), (int)(cr[js] >> 16));
        } else {
#pragma unroll
            for (int j = 0; j < JE; j++) xs[tid + j * COMB_THREADS] = mn == INF_F ? 0.f : __builtin_amdgcn_exp2f(mn - x[j]);
            __syncthreads();
            // per-emission sums in fixed (input) order
            float lsum = 0.f;
#pragma unroll
            for (int js = 0; js < JS; js++) {
                sd[js] = slot_sum(xs, (int)(cr[js] & 0xFFFFu), (int)(cr[js] >> 16));
                lsum += sd[js];
            }
            tot = block_sum256(lsum, redsum);
        }
        const bool dead = mn == INF_F;
        const float logtot = __builtin_amdgcn_logf(tot);
        if (tid == 0)
            a.sum_output[(size_t)t * B + b] = dead ? 0.f : (float)(((double)(mn - logtot) + offs) * (double)LN2);
        const float inv = dead ? 0.f : psign / tot;
        float* cprow = cpbase + (size_t)t * DP;
#pragma unroll
        for (int js = 0; js < JS; js++) {
            const int d = tid + js * COMB_THREADS;
            if (d < D) {
                float v;
                if (prob) v = sd[js] * inv;
                else if (NEGLOG) v = dead ? INF_F : neg_log_value(ls[js], mn, logtot);
                else v = (dead || sd[js] == 0.f) ? INF_F : (logtot - __builtin_amdgcn_logf(sd[js])) * LN2;
                store_agent(cprow + d, v);
            }
        }
    }
    wait_stores();
    __syncthreads();
    if (tid == 0) store_agent(flag, 1);
}

// Rows [row0, row1) of the tensor in memory order are this group's (frames [t0, ...) of all
// sequences in layout 0, of sequence bg in layout 1); this job writes the spans job, job + nW,
// job + 2 nW, ... of the group: jobs that run side by side then write neighbouring spans, i.e. one
// contiguous window of memory that moves on as they move on (consecutive spans per job -- a window
// of scattered pieces -- measured slower).  All a job needs from memory is fetched up front in two
// rounds -- the records of the sequences whose rows its spans cut, their flags and the slot ranges
// of its pieces of those rows; then emission index and posterior of every slot in those ranges
// (into registers) -- so that the spans themselves go out back to back: scatter the values that
// fall into the span into the LDS image, read it back in 16-byte chunks, store, clear.  A span of
// FLAT_W <= F floats cuts at most two rows.
template <bool SYNC>
__device__ __forceinline__ void flat_write(const FlatArgs& fa, const long long row0, const long long row1, const int t0, const int bg,
                                           const int job, float4a* img4, int* s_row, long long* s_off) {
    const CombArgs& a = fa.c;
    const int tid = threadIdx.x;
    const int T = a.T, B = a.B, F = a.F;
    const long long g0 = row0 * F + fa.shift, g1 = row1 * F + fa.shift;     // in the line-aligned view (base = out - shift)
    const long long first = g0 & ~31LL;                                     // first span of the group
    const int group_spans = (int)((g1 - first + FLAT_W - 1) / FLAT_W);
    if (job >= group_spans) return;
    const int nspans = min(FLAT_KMAX, (group_spans - job + fa.nW - 1) / fa.nW);
#ifdef I6_TRACE
    const bool traced = (blockIdx.x % 997) == 5 && blockIdx.x / 997 < 60 && tid == 0;
    unsigned long long* tr = g_trace + 2048 + (blockIdx.x / 997) * 16;
    if (traced) { tr[0] = wall_clock64(); tr[15] = blockIdx.x; }
#endif
    float* image = (float*)img4;
    const float hole = a.out_mode != I6FBW_OUT_NEG_LOG ? 0.f : INF_F;
    const float4a hole4 = {hole, hole, hole, hole};
    static_assert(FLAT_W / 4 == 2 * COMB_THREADS, "two chunks per thread");
    img4[tid] = hole4;
    img4[tid + COMB_THREADS] = hole4;
    // per (span, first or second row it cuts): what the piece is made of (-1 no such piece, 0 holes
    // only, 1 compact posteriors, 2 NaN, 3 left to fbw_combine), its place in the span, and for kind 1
    // the slot range of the piece and where the slots' emission indices and values are
    int* s_kind = s_row;
    int* s_lo = s_row + 2 * FLAT_KMAX;
    int* s_hi = s_row + 4 * FLAT_KMAX;
    int* s_at = s_row + 6 * FLAT_KMAX;      // position of emission 0 of the row relative to the span (may be negative)
    int* s_p0 = s_row + 8 * FLAT_KMAX;      // piece [s_p0, s_p1) of the span
    int* s_p1 = s_row + 10 * FLAT_KMAX;
    long long* s_de = s_off;
    long long* s_cp = s_off + 2 * FLAT_KMAX;
    if (tid < 2 * nspans) {
        const int k = tid >> 1;
        const long long span0 = first + (long long)(job + k * fa.nW) * FLAT_W;
        const long long lo = max(span0, g0), hi = min(span0 + FLAT_W, g1);
        // (a group holds fewer than 2^31 floats: the host sees to that)
        const unsigned rr = (unsigned)(lo - g0) / (unsigned)F + (tid & 1);          // row within the group
        const long long rbeg = g0 + (long long)rr * F;
        const long long pl = max(lo, rbeg), ph = min(hi, rbeg + F);
        int kind = -1, s0 = 0, s1 = 0;
        if (pl < ph) {
            const int t = fa.layout == 0 ? t0 + (int)(rr / (unsigned)B) : t0 + (int)rr;
            const int b = fa.layout == 0 ? (int)(rr % (unsigned)B) : bg;
            // everything is requested before the first answer is looked at
            const SeqMeta m = a.meta[b];
            const int* wp = fa.wpfx + (size_t)b * fa.wpfx_stride;
            const int w0 = wp[(int)(pl - rbeg) >> 5], w1 = wp[((int)(ph - rbeg) + 31) >> 5];
            const int* flag = fa.cflag + (size_t)b * ((T + FLAT_TCF - 1) / FLAT_TCF) + t / FLAT_TCF;
            const int f0 = load_agent(flag);
            kind = 0;
            if (t < m.L) {
                if (seq_error(m) < 0) kind = 2;
                else if (m.n_edges == 0) kind = 0;
                else if (!flat_fast(m)) kind = 3;
                else {
                    s0 = w0; s1 = w1;
                    const long long goff = slot_off(m.edge_begin, b);
                    s_de[tid] = goff;
                    s_cp[tid] = (long long)T * goff + (long long)t * m.DP;
                    kind = (f0 >= 1 || spin_until_ge(flag, 1, a.sync)) && load_agent(flag) == 1 ? 1 : 2;
                }
            }
        }
        s_kind[tid] = kind; s_lo[tid] = s0; s_hi[tid] = s1;
        s_at[tid] = (int)(rbeg - span0); s_p0[tid] = (int)(pl - span0); s_p1[tid] = (int)(ph - span0);
    }
    __syncthreads();
#ifdef I6_TRACE
    if (traced) tr[1] = wall_clock64();
#endif
    // Slots of the pieces -> registers.  Piece i belongs to the LP lanes from i * LP on; each of them
    // takes every LP-th slot of the piece, up to NSP of them: position within the span (-1: none)
    // and value.  With LP = 16 lanes per piece the 16 pieces of the job are fetched in one round, which
    // covers pieces of up to 128 slots; a job with fuller pieces (sequences that use more than a
    // sixteenth of the emissions) takes its spans four or two at a time with 32 or 64 lanes per piece,
    // and what is still left of a piece then is fetched while its span is built.
    constexpr int LP = COMB_THREADS / (2 * FLAT_KMAX), NSP = 8;
    static_assert(LP * 2 * FLAT_KMAX == COMB_THREADS && LP >= 1, "lanes per piece");
    int q[NSP];
    float v[NSP];
    // pieces 2 * k0 ... of the job, lp lanes each
    auto fetch_pieces = [&](const int k0, const int lp) {
        const int mine = 2 * k0 + tid / lp, ln = tid % lp;          // my piece, my lane within it
        const bool have = mine < 2 * nspans && s_kind[mine] == 1;
        // (all loads are issued before the first result is used: index and value do not depend on each other)
        const int s0 = have ? s_lo[mine] : 0, s1 = have ? s_hi[mine] : 0;
        const int* de = a.demis + (have ? s_de[mine] : 0);
        const float* cprow = fa.cp + (have ? s_cp[mine] : 0);
#pragma unroll
        for (int n = 0; n < NSP; n++) {
            const int sl = s0 + ln + n * lp;
            q[n] = -1; v[n] = 0.f;
            if (sl < s1) { q[n] = de[sl]; v[n] = load_agent(cprow + sl); }
        }
        const int at = have ? s_at[mine] : 0, p0 = have ? s_p0[mine] : 0, p1 = have ? s_p1[mine] : 0;
#pragma unroll
        for (int n = 0; n < NSP; n++) {
            if (q[n] >= 0) {
                const int pos = at + q[n];
                q[n] = (pos >= p0 && pos < p1) ? pos : -1;
            }
        }
    };
    float* dst0 = (a.out - fa.shift) + first;
    // span k of the job: mine = whether my registers hold values of it, held = slots per piece that the registers cover
    auto emit_span = [&](const int k, const bool mine, const int held, const bool check_rest) {
        const long long span0 = first + (long long)(job + k * fa.nW) * FLAT_W;
        const int ka = s_kind[2 * k], kb = s_kind[2 * k + 1];
        // Spans that need care: cut by an end of the group, or holding a piece that is constant (NaN) or
        // not written here.  All others -- nearly all -- take the short way: a handful of LDS writes, two
        // LDS reads, two stores.
        const bool special = span0 < g0 || span0 + FLAT_W > g1 || ka >= 2 || kb >= 2;
        if (special) {
#pragma unroll
            for (int w = 0; w < 2; w++) {
                const int kind = w ? kb : ka;
                if (kind < 2) continue;
                const float c = kind == 2 ? __builtin_nanf("") : __uint_as_float(FLAT_SKIP);
                for (int i = s_p0[2 * k + w] + tid; i < s_p1[2 * k + w]; i += COMB_THREADS) image[i] = c;
            }
            // elements of the span outside the group belong to the neighbouring group
            for (int i = tid; i < (int)(g0 - span0); i += COMB_THREADS) image[i] = __uint_as_float(FLAT_SKIP);
            for (int i = (int)max(0LL, g1 - span0) + tid; i < FLAT_W; i += COMB_THREADS) image[i] = __uint_as_float(FLAT_SKIP);
        }
        // the image holds holes everywhere else (see below); now my values of this span
        if (mine) {
#pragma unroll
            for (int n = 0; n < NSP; n++)
                if (q[n] >= 0) image[q[n]] = v[n];
        }
        if (check_rest) {
            for (int w = 0; w < 2; w++) {
                const int i = 2 * k + w;
                if (s_kind[i] != 1) continue;
                for (int sl = s_lo[i] + held + tid; sl < s_hi[i]; sl += COMB_THREADS) {
                    const int pos = s_at[i] + a.demis[s_de[i] + sl];
                    if (pos >= s_p0[i] && pos < s_p1[i]) image[pos] = load_agent(fa.cp + s_cp[i] + sl);
                }
            }
        }
        lds_barrier();
        float4a c4[2];
#pragma unroll
        for (int u = 0; u < 2; u++) c4[u] = img4[tid + u * COMB_THREADS];
        float* d0 = dst0 + (size_t)(job + k * fa.nW) * FLAT_W + 4 * tid;
        if (!special) {
#pragma unroll
            for (int u = 0; u < 2; u++) I6_ROW_STORE(c4[u], (float4a*)(d0 + 4 * u * COMB_THREADS));
        } else {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                float* d = d0 + 4 * u * COMB_THREADS;
                const bool whole = __float_as_uint(c4[u].x) != FLAT_SKIP && __float_as_uint(c4[u].y) != FLAT_SKIP &&
                                   __float_as_uint(c4[u].z) != FLAT_SKIP && __float_as_uint(c4[u].w) != FLAT_SKIP;
                if (whole) I6_ROW_STORE(c4[u], (float4a*)d);
                else {
                    if (__float_as_uint(c4[u].x) != FLAT_SKIP) d[0] = c4[u].x;
                    if (__float_as_uint(c4[u].y) != FLAT_SKIP) d[1] = c4[u].y;
                    if (__float_as_uint(c4[u].z) != FLAT_SKIP) d[2] = c4[u].z;
                    if (__float_as_uint(c4[u].w) != FLAT_SKIP) d[3] = c4[u].w;
                }
            }
        }
        // every thread clears the chunks it has read: holes everywhere again
        img4[tid] = hole4;
        img4[tid + COMB_THREADS] = hole4;
        lds_barrier();
    };
    int fullest = 0;
    for (int i = 0; i < 2 * nspans; i++) if (s_kind[i] == 1) fullest = max(fullest, s_hi[i] - s_lo[i]);
    if (fullest <= LP * NSP) {
        fetch_pieces(0, LP);
#ifdef I6_TRACE
        if (traced) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); tr[2] = wall_clock64(); }
#endif
#pragma unroll
        for (int k = 0; k < FLAT_KMAX; k++) {
            if (k >= nspans) break;
            emit_span(k, ((tid / LP) >> 1) == k, LP * NSP, false);
#ifdef I6_TRACE
            if (traced) tr[3 + k] = wall_clock64();
#endif
        }
    } else {
        const int lp = fullest <= 2 * LP * NSP ? 2 * LP : 4 * LP;
        const int per_round = COMB_THREADS / (2 * lp);          // spans whose pieces one round of registers holds
        for (int k0 = 0; k0 < nspans; k0 += per_round) {
            fetch_pieces(k0, lp);
            for (int k = k0; k < min(nspans, k0 + per_round); k++)
                emit_span(k, ((tid / lp) >> 1) == k - k0, lp * NSP, fullest > lp * NSP);
        }
    }
#ifdef I6_TRACE
    if (traced) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); tr[12] = wall_clock64(); }
#endif
}

// (the -log instance needs a few registers more for its sums in log space: six workgroups per compute unit)
template <bool SYNC, bool NEGLOG>
__global__ __launch_bounds__(COMB_THREADS, NEGLOG ? (I6_FLAT_OCC < 6 ? I6_FLAT_OCC : 6) : I6_FLAT_OCC) void fbw_flat(FlatArgs fa) {
    // image of a write job; staging area of a posterior job (the scores of the edges of its frames)
    __shared__ float4a img4[FLAT_TCF * FLAT_EDGES / 4];
    static_assert(FLAT_TCF * FLAT_EDGES >= FLAT_W, "the image fits");
    __shared__ float redmin[COMB_THREADS / 64];
    __shared__ float redsum[COMB_THREADS / 64];
    __shared__ int s_kind[12 * FLAT_KMAX];
    __shared__ long long s_off[4 * FLAT_KMAX];
    static_assert(FLAT_W >= COMB_FAST_EDGES, "the staging area of a posterior job lies in the image");
    const int B = fa.c.B, T = fa.c.T;
    const int n = (T + TC - 1) / TC;
    // job of this workgroup
    constexpr int NQ = TC / FLAT_TCF;           // posterior jobs per strip of a sequence
    int i, b = -1, job = -1, qf = 0;            // job >= 0: write job number within its group; qf: which part of the strip
    const int blk = blockIdx.x;
    if (blk < fa.ahead * B * NQ) { i = blk / (B * NQ); b = (blk / NQ) % B; qf = blk % NQ; }
    else {
        const int x = blk - fa.ahead * B * NQ;
        const int G = fa.nW + (fa.layout == 0 ? B : 1) * NQ;
        const int u = x / G, r = x % G;
        if (fa.layout == 0) { i = u; if (r < fa.nW) job = r; else { b = (r - fa.nW) / NQ; qf = (r - fa.nW) % NQ; i += fa.ahead; } }
        else { i = u / B; b = u % B; if (r < fa.nW) job = r; else { qf = r - fa.nW; i += fa.ahead; } }
    }
#ifdef I6_TRACE
    if (blk == 0 && threadIdx.x == 0) g_trace[2040] = wall_clock64();
    trace_corun(3100);
#endif
    if (i >= n) return;
    // middle: where the two recursions meet -- of the longest sequence (rows of all sequences of a
    // frame lie side by side) or of this sequence
    const int Lmid = fa.layout == 0 ? fa.c.sync[6] : fa.c.meta[b].L;
    const int strip = middle_out(i, n, min(n - 1, (Lmid / 2) / TC));
    if (job < 0) {
        flat_post<SYNC, NEGLOG>(fa, b, strip * TC + qf * FLAT_TCF, (float*)img4, redmin, redsum, s_kind);
        return;
    }
    const long long row0 = fa.layout == 0 ? (long long)strip * TC * B : (long long)b * T + strip * TC;
    const long long row1 = fa.layout == 0 ? (long long)min(T, strip * TC + TC) * B : (long long)b * T + min(T, strip * TC + TC);
    flat_write<SYNC>(fa, row0, row1, strip * TC, b, job, img4, s_kind, s_off);
}

// Status of a call in two ints {code, sequence}: the first sequence with a reported problem, else a
// timeout of the hand-off between kernels, else ok.  One workgroup.
__global__ __launch_bounds__(256) void fbw_status_reduce(const SeqMeta* meta, int B, const int* sync, int* out2) {
    __shared__ int first_bad;
    if (threadIdx.x == 0) first_bad = 0x7fffffff;
    __syncthreads();
    for (int b = threadIdx.x; b < B; b += 256)
        if (meta[b].err < 0 || meta[b].errA < 0 || meta[b].errB < 0) atomicMin(&first_bad, b);
    __syncthreads();
    if (threadIdx.x == 0) {
        int code = sync[0] ? I6FBW_ERR_TIMEOUT : I6FBW_OK, seq = -1;
        if (first_bad != 0x7fffffff) {
            const SeqMeta& m = meta[first_bad];
            code = m.err < 0 ? m.err : (m.errA < 0 ? m.errA : m.errB);
            seq = first_bad;
        }
        out2[0] = code; out2[1] = seq;
    }
}

// Check that two streams really run at the same time (see runs_beside).
__device__ int g_selftest[4];
__global__ void fbw_selftest_wait() {
    if (threadIdx.x == 0) {
        int seen = 0;
        for (int n = 0; n < (1 << 18) && !seen; n++) { seen = load_agent(&g_selftest[0]); __builtin_amdgcn_s_sleep(8); }
        store_agent(&g_selftest[1], seen ? 1 : 2);
    }
}
__global__ void fbw_selftest_set(int v) { if (threadIdx.x == 0) store_agent(&g_selftest[0], v); }

// Holds back the combine kernel (next on the same stream) until every workgroup of the recursion
// kernel has been placed on the machine: combine workgroups wait for recursion progress while
// they occupy LDS and wave slots, so they must not be able to keep a recursion workgroup out.
__global__ __launch_bounds__(64) void fbw_gate(int* sync, int need) {
    if (threadIdx.x == 0) spin_until_ge(sync + 1, need, sync);
}

// Rows of frames t >= seq_len (all rows if seq_len is outside [1, T]): out = hole, sum_output = 0
// (fbw_op.cu:120-128,366-369).  They depend on nothing but seq_lens, so this kernel runs beside
// the edge preparation.  Sequences that turn out to have no edges or a problem are written by
// fbw_combine.
__global__ __launch_bounds__(COMB_THREADS) void fbw_padfill(const int32_t* seq_lens, int T, int B, int F, int out_mode,
                                                            float* out, long long ost_t, long long ost_b, float* sum_output) {
    const int b = blockIdx.x, t0 = blockIdx.y * TC;
    const unsigned sl = (unsigned)seq_lens[b];
    const int L = (sl >= 1u && sl <= (unsigned)T) ? (int)sl : 0;
    const int t1 = min(T, t0 + TC);
    const float hole = out_mode != I6FBW_OUT_NEG_LOG ? 0.f : INF_F;
    for (int t = max(t0, L); t < t1; t++) {
        stream_const_row(out + t * ost_t + b * ost_b, F, hole);
        if (threadIdx.x == 0) sum_output[(size_t)t * B + b] = 0.f;
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
constexpr int MAX_DEVICES = 64;

thread_local hipError_t g_last_hip_error = hipSuccess;

#define HIP_TRY(expr)                                              \
    do {                                                           \
        hipError_t e_ = (expr);                                    \
        if (e_ != hipSuccess) { g_last_hip_error = e_; return I6FBW_ERR_LAUNCH; } \
    } while (0)

// Library-owned streams and events of one device.  A large call keeps the edge preparation, the
// gather and the dense write on the caller's stream and runs the padding fill and the recursion
// beside them on two streams of its own; the kernels that run at the same time feed each other
// through flags in memory.
struct Pipeline {
    std::mutex mu;            // calls on one device are serialised (they share its streams and events); devices are independent
    bool attr_ready = false;  // kernel attributes set, device facts read
    bool ready = false;       // streams and events created
    hipStream_t sP = nullptr, sR = nullptr;
    hipEvent_t start = nullptr, fork = nullptr, gathered = nullptr, doneP = nullptr, doneR = nullptr;
    int n_cu = 256;
    int dense_regs = 0;       // vector registers per lane of fbw_recurse_dense<true>, as built
    // caller streams that were checked against the recursion stream: do kernels on the two run at
    // the same time?
    std::vector<std::pair<hipStream_t, bool>> checked;
    void* static_ws = nullptr;   // this device's copy of g_static_workspace (i6fbw_run_static)
};
Pipeline g_pipe[MAX_DEVICES];
std::mutex g_mutex;           // process-wide settings and the stage profile

// Built-in workspace of i6fbw_run_static, for callers that cannot allocate device memory.  Every
// device the library runs on holds its own copy for the life of the process; host code reaches it
// only through the address hipGetSymbolAddress returns for the current device (Pipeline::static_ws).
static __device__ __align__(256) unsigned char g_static_workspace[I6FBW_STATIC_WORKSPACE_BYTES];

// LDS of a preparation workgroup: sort keys, emission bitmap and its prefix counts
size_t prep_lds_bytes(int F) { return (size_t)(EB_MAX + PREP_AUX_WORDS) * 4 + (F <= F_BITMAP_MAX ? (size_t)((F + 31) >> 5) * 8 : 0); }

// 1024-thread workgroups sort fastest, but only two of them fit on a compute unit: batches that
// would need a second round of them take 512-thread workgroups, four to a unit.
void launch_prepare(const Pipeline& P, const PrepArgs& pa, hipStream_t s) {
    const size_t lds = prep_lds_bytes(pa.F);
    // 512 threads: four workgroups per compute unit for large batches (one round instead of two), and for sequences of up
    // to 512 edges on average, which have no work for more (fewer waves at every barrier: 50 x 2 x 10 0.058 -> 0.052 ms per
    // call, 500 x 32 x 264 0.178 -> 0.173; 750 edges per sequence: no difference; 256 threads: slower from 380 edges on)
    if (3 * pa.B > 2 * P.n_cu || (long long)pa.E <= 512LL * pa.B) hipLaunchKernelGGL(fbw_prepare<512>, dim3(3, pa.B), dim3(512), lds, s, pa);
    else hipLaunchKernelGGL(fbw_prepare<1024>, dim3(3, pa.B), dim3(1024), lds, s, pa);
}

// The dense writers, in the instance for the output mode (NEGLOG: the -log output, summed in log space)
// (the row writer proper: first the instance for small sequences -- most batches are nothing else -- then the general
// one for the rest; rows too long for the LDS image, and the sequences fbw_flat leaves over, are the general one's alone)
// (LDS of the small-sequence instance where it takes COMB_BATCH frames together: that many row images and staging areas)
size_t comb_batch_lds_bytes(int F) { return (size_t)COMB_BATCH * ((size_t)(((F + 32 + 3) >> 2) * 16) + (size_t)COMB_BATCH_EDGES * 4); }
template <bool SYNC>
void launch_combine(const bool neglog, const dim3 grid, const size_t lds, hipStream_t s, CombArgs ca) {
    if (!ca.direct_only && !ca.tile_w) {
        size_t lds_s = lds;
        if (ca.F <= COMB_BATCH_F) { ca.batch_frames = 1; lds_s = std::max(lds, comb_batch_lds_bytes(ca.F)); }      // (both instances: it decides which takes a sequence)
        CombArgs cs = ca;
        if (neglog) hipLaunchKernelGGL((fbw_combine<SYNC, true, true>), grid, dim3(COMB_THREADS), lds_s, s, cs);
        else hipLaunchKernelGGL((fbw_combine<SYNC, false, true>), grid, dim3(COMB_THREADS), lds_s, s, cs);
        ca.small_elsewhere = 1;
    }
    if (neglog) hipLaunchKernelGGL((fbw_combine<SYNC, true, false>), grid, dim3(COMB_THREADS), lds, s, ca);
    else hipLaunchKernelGGL((fbw_combine<SYNC, false, false>), grid, dim3(COMB_THREADS), lds, s, ca);
}
template <bool SYNC>
void launch_flat(const bool neglog, const dim3 grid, hipStream_t s, const FlatArgs& fa) {
    if (neglog) hipLaunchKernelGGL((fbw_flat<SYNC, true>), grid, dim3(COMB_THREADS), 0, s, fa);
    else hipLaunchKernelGGL((fbw_flat<SYNC, false>), grid, dim3(COMB_THREADS), 0, s, fa);
}

// Device facts and kernel attributes; creates nothing (i6fbw_run_static stops here).
int device_init(Pipeline& p) {
    if (p.attr_ready) return I6FBW_OK;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipDeviceGetAttribute(&p.n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    HIP_TRY(hipFuncSetAttribute((const void*)fbw_recurse_dense<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(float) * REC_LDS_FLOATS_F32));
    HIP_TRY(hipFuncSetAttribute((const void*)fbw_recurse_dense<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(float) * REC_LDS_FLOATS_F32));
    HIP_TRY(hipFuncSetAttribute((const void*)fbw_prepare<1024>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)prep_lds_bytes(F_BITMAP_MAX)));
    HIP_TRY(hipFuncSetAttribute((const void*)fbw_prepare<512>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)prep_lds_bytes(F_BITMAP_MAX)));
    for (const void* k : {(const void*)fbw_combine<true, false, false>, (const void*)fbw_combine<false, false, false>,
                          (const void*)fbw_combine<true, true, false>, (const void*)fbw_combine<false, true, false>,
                          (const void*)fbw_combine<true, false, true>, (const void*)fbw_combine<false, false, true>,
                          (const void*)fbw_combine<true, true, true>, (const void*)fbw_combine<false, true, true>})
        HIP_TRY(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256));
    hipFuncAttributes attr;
    HIP_TRY(hipFuncGetAttributes(&attr, (const void*)fbw_recurse_dense<true>));
    p.dense_regs = attr.numRegs;
    // address of the current device's copy of the built-in workspace
    HIP_TRY(hipGetSymbolAddress(&p.static_ws, HIP_SYMBOL(g_static_workspace)));
    p.attr_ready = true;
    return I6FBW_OK;
}

int pipeline_init(Pipeline& p) {
    if (p.ready) return I6FBW_OK;
    { int rc = device_init(p); if (rc != I6FBW_OK) return rc; }
    // default priority on purpose
    HIP_TRY(hipStreamCreateWithFlags(&p.sP, hipStreamNonBlocking));
    HIP_TRY(hipStreamCreateWithFlags(&p.sR, hipStreamNonBlocking));
    for (hipEvent_t* e : {&p.start, &p.fork, &p.gathered, &p.doneP, &p.doneR})
        HIP_TRY(hipEventCreateWithFlags(e, hipEventDisableTiming));
    p.ready = true;
    return I6FBW_OK;
}

// In the overlapped schedule the recursion kernel (library stream) waits in memory for kernels that
// the caller's stream starts after it.  That only works if the two streams are served at the same
// time; the first large call on a stream checks it with a bounded handshake between two one-wave
// kernels (this synchronises the stream once), and the single-stream schedule is used if the waiter
// never sees the flag (e.g. both streams mapped to one hardware queue, or a serialising profiler).
int runs_beside(Pipeline& p, hipStream_t s, bool* yes) {
    for (const auto& c : p.checked)
        if (c.first == s) { *yes = c.second; return I6FBW_OK; }
    fbw_selftest_set<<<1, 64, 0, s>>>(0);
    HIP_TRY(hipStreamSynchronize(s));
    fbw_selftest_wait<<<1, 64, 0, p.sR>>>();
    fbw_selftest_set<<<1, 64, 0, s>>>(1);
    HIP_TRY(hipStreamSynchronize(p.sR));
    HIP_TRY(hipStreamSynchronize(s));
    int result[4] = {0, 0, 0, 0};
    HIP_TRY(hipMemcpyFromSymbol(result, HIP_SYMBOL(g_selftest), sizeof(result)));
    *yes = result[1] == 1;
    if (p.checked.size() >= 64) p.checked.clear();
    p.checked.emplace_back(s, *yes);
    return I6FBW_OK;
}

// A hand-off timeout means that kernels which should have run side by side did not: the answers
// cached per stream are dropped, and the next large call on a stream checks again.
void forget_stream_checks() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return;
    std::lock_guard<std::mutex> lock(g_pipe[dev].mu);
    g_pipe[dev].checked.clear();
}

// Stage timing: event pairs around every launch of a stage, on the stream it runs on.
struct Profile {
    std::atomic<bool> on{false};
    static constexpr int MAXPAIR = 8192;
    int n_pairs = 0, n_calls = 0;
    hipEvent_t a[MAXPAIR], b[MAXPAIR];
    int stage[MAXPAIR];
    int n_created = 0;
};
Profile g_prof;

struct StageTimer {
    int idx = -1;
    hipStream_t stream;
    StageTimer(int stage, hipStream_t st, bool enabled) : stream(st) {
        if (!enabled) return;
        std::lock_guard<std::mutex> lock(g_mutex);      // the profile is shared by all devices
        if (g_prof.n_pairs >= Profile::MAXPAIR) return;
        if (g_prof.n_pairs >= g_prof.n_created) {
            if (hipEventCreate(&g_prof.a[g_prof.n_created]) != hipSuccess) return;
            if (hipEventCreate(&g_prof.b[g_prof.n_created]) != hipSuccess) return;
            g_prof.n_created++;
        }
        idx = g_prof.n_pairs++;
        g_prof.stage[idx] = stage;
        (void)hipEventRecord(g_prof.a[idx], stream);
    }
    ~StageTimer() {
        if (idx >= 0) (void)hipEventRecord(g_prof.b[idx], stream);
    }
};

int row_misalign_host(const float* p) { return (int)(((uintptr_t)p >> 2) & 31); }
size_t comb_lds_bytes(int F) { return (size_t)(((F + 32 + 3) >> 2) * 16) + (size_t)COMB_XS * 4; }
constexpr int COMB_TILE_W = 12288;     // floats of a row that go through LDS at a time when the row does not fit: three workgroups per unit

// schedule: -1 by problem size, 0 single stream, 1 overlapped; I6FBW_OVERLAP=0/1 sets the initial value
std::atomic<int> g_all_frames_default{0};      // i6fbw_set_band(0), kept for callers of earlier versions: every call as with I6FBW_IN_ALL_FRAMES
std::atomic<int> g_overlap_mode{[] {
    const char* e = getenv("I6FBW_OVERLAP");
    return e ? (e[0] == '0' ? 0 : 1) : -1;
}()};

// dense writer: -1 by problem (flat spans where the layout allows it and the stages overlap), 0 always row by row,
// 1 flat wherever the layout allows it; I6FBW_DENSE_WRITER=rows|flat sets the initial value
std::atomic<int> g_writer_mode{[] {
    const char* e = getenv("I6FBW_DENSE_WRITER");
    return e ? (e[0] == 'r' ? 0 : 1) : -1;
}()};

std::atomic<int> g_last_writer{0};     // writer of the most recent i6fbw_run of the process: 0 rows, 1 flat spans

// Status reports that travel to the host without a wait: per device a ring of pinned {code, seq}
// slots, each with the event that follows its copy on the caller's stream.
struct StatusRing {
    static constexpr int SLOTS = 64;
    int* host = nullptr;                 // SLOTS x 2 ints, pinned
    hipEvent_t ev[SLOTS] = {};
    bool used[SLOTS] = {};
    int next = 0;
    int held_code = I6FBW_OK, held_seq = -1;     // first problem seen and not yet handed to the caller
};
StatusRing g_status[MAX_DEVICES];

// takes the result out of slot i (its event has completed or is waited for here); false if the
// report is still on its way
bool status_collect(StatusRing& r, int i, bool wait) {
    if (!r.used[i]) return true;
    if (wait) { if (hipEventSynchronize(r.ev[i]) != hipSuccess) return false; }
    else if (hipEventQuery(r.ev[i]) != hipSuccess) return false;
    r.used[i] = false;
    const int code = r.host[2 * i], seq = r.host[2 * i + 1];
    if (code != I6FBW_OK && r.held_code == I6FBW_OK) { r.held_code = code; r.held_seq = seq; }
    return true;
}

// how the bindings report device-side problems: 0 not at all, 1 by waiting for every call, 2 without
// waiting, at a later call; I6FBW_STATUS=off|sync|deferred sets the initial value (I6FBW_ASYNC=1: off)
std::atomic<int> g_status_mode{[] {
    const char* e = getenv("I6FBW_STATUS");
    if (e) return e[0] == 'o' ? 0 : (e[0] == 's' ? 1 : 2);
    const char* a = getenv("I6FBW_ASYNC");
    return (a && a[0] == '1') ? 0 : 2;
}()};

int run_impl(const float* am, int64_t am_stride_t, int64_t am_stride_b, int input_flags,
             const int32_t* edges, int64_t edge_row_stride, const float* weights, const int32_t* start_end,
             int64_t se_row_stride, const int32_t* seq_lens, int T, int B, int F, int E, int n_states,
             int out_mode, float* out, int64_t out_stride_t, int64_t out_stride_b, float* sum_output,
             void* workspace, size_t workspace_bytes, void* stream_, const bool static_call);

}  // namespace

extern "C" {

int i6fbw_workspace_size(int T, int B, int F, int E, int n_states, size_t* bytes) {
    if (!bytes || T <= 0 || B <= 0 || F <= 0 || E < 0 || n_states <= 0) return I6FBW_ERR_INVALID_ARGUMENT;
    *bytes = make_layout(T, B, E, F).total;
    return I6FBW_OK;
}

int i6fbw_run(const float* am, int64_t am_stride_t, int64_t am_stride_b, const int32_t* edges, int64_t edge_row_stride,
              const float* weights, const int32_t* start_end, int64_t se_row_stride, const int32_t* seq_lens, int T,
              int B, int F, int E, int n_states, int out_mode, float* out, float* sum_output, void* workspace,
              size_t workspace_bytes, void* stream_) {
    return i6fbw_run_strided(am, am_stride_t, am_stride_b, 0, edges, edge_row_stride, weights, start_end, se_row_stride,
                             seq_lens, T, B, F, E, n_states, out_mode, out, (int64_t)B * F, (int64_t)F, sum_output,
                             workspace, workspace_bytes, stream_);
}

int i6fbw_run_strided(const float* am, int64_t am_stride_t, int64_t am_stride_b, int input_flags,
                      const int32_t* edges, int64_t edge_row_stride, const float* weights, const int32_t* start_end,
                      int64_t se_row_stride, const int32_t* seq_lens, int T, int B, int F, int E, int n_states,
                      int out_mode, float* out, int64_t out_stride_t, int64_t out_stride_b, float* sum_output,
                      void* workspace, size_t workspace_bytes, void* stream_) {
    return run_impl(am, am_stride_t, am_stride_b, input_flags, edges, edge_row_stride, weights, start_end,
                    se_row_stride, seq_lens, T, B, F, E, n_states, out_mode, out, out_stride_t, out_stride_b, sum_output,
                    workspace, workspace_bytes, stream_, false);
}

int i6fbw_run_static(const float* am, int64_t am_stride_t, int64_t am_stride_b, const int32_t* edges, int64_t edge_row_stride,
                     const float* weights, const int32_t* start_end, int64_t se_row_stride, const int32_t* seq_lens, int T,
                     int B, int F, int E, int n_states, int out_mode, float* out, float* sum_output, void* stream_) {
    // workspace == nullptr: run_impl takes the current device's built-in buffer
    return run_impl(am, am_stride_t, am_stride_b, 0, edges, edge_row_stride, weights, start_end, se_row_stride, seq_lens,
                    T, B, F, E, n_states, out_mode, out, (int64_t)B * F, (int64_t)F, sum_output, nullptr, 0, stream_, true);
}

int i6fbw_static_workspace(void** workspace, size_t* bytes) {
    if (!workspace || !bytes) return I6FBW_ERR_INVALID_ARGUMENT;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return I6FBW_ERR_INVALID_ARGUMENT;
    Pipeline& P = g_pipe[dev];
    std::lock_guard<std::mutex> lock(P.mu);
    { int rc = device_init(P); if (rc != I6FBW_OK) return rc; }
    *workspace = P.static_ws; *bytes = I6FBW_STATIC_WORKSPACE_BYTES;
    return I6FBW_OK;
}

}  // extern "C"

namespace {
// Body of i6fbw_run_strided and i6fbw_run_static.  static_call: the workspace is the device's
// built-in buffer, and nothing may be allocated or created -- no library streams or events, no
// stage timers: the stages run one after the other on the caller's stream.
int run_impl(const float* am, int64_t am_stride_t, int64_t am_stride_b, int input_flags,
             const int32_t* edges, int64_t edge_row_stride, const float* weights, const int32_t* start_end,
             int64_t se_row_stride, const int32_t* seq_lens, int T, int B, int F, int E, int n_states,
             int out_mode, float* out, int64_t out_stride_t, int64_t out_stride_b, float* sum_output,
             void* workspace, size_t workspace_bytes, void* stream_, const bool static_call) {
    if (T <= 0 || B <= 0 || F <= 0 || E < 0 || n_states <= 0) return I6FBW_ERR_INVALID_ARGUMENT;
    if (!am || !start_end || !seq_lens || !out || !sum_output || (!workspace && !static_call)) return I6FBW_ERR_INVALID_ARGUMENT;
    if (E > 0 && (!edges || !weights)) return I6FBW_ERR_INVALID_ARGUMENT;
    if (out_mode != I6FBW_OUT_NEG_LOG && out_mode != I6FBW_OUT_PROB && out_mode != I6FBW_OUT_NEG_PROB) return I6FBW_ERR_INVALID_ARGUMENT;
    if (input_flags & ~(I6FBW_IN_LOG_PROBS | I6FBW_IN_ALL_FRAMES)) return I6FBW_ERR_INVALID_ARGUMENT;
    input_flags |= g_all_frames_default.load();
    if (out_stride_t < 0 || out_stride_b < 0) return I6FBW_ERR_INVALID_ARGUMENT;
    if (((uintptr_t)workspace & 255) != 0) return I6FBW_ERR_INVALID_ARGUMENT;
    if (B > 65535 || (T + TC - 1) / TC > 65535) return I6FBW_ERR_INVALID_ARGUMENT;   // grid limits
    const Layout l = make_layout(T, B, E, F);
    if (static_call) {
        if (l.total > (size_t)I6FBW_STATIC_WORKSPACE_BYTES) return I6FBW_ERR_STATIC_WORKSPACE;
    } else if (workspace_bytes < l.total) return I6FBW_ERR_WORKSPACE_TOO_SMALL;
    // too many emission classes for the LDS bitmap of the preparation: every sequence takes the general path
    const bool f_too_large = F > F_BITMAP_MAX;
    // rows too long for the LDS image of the dense write go through it in tiles; so do rows of more
    // than two tiles that would still fit (the smaller image leaves room for three workgroups on a
    // compute unit instead of one or two: 1-2 % faster)
    const bool tiled = comb_lds_bytes(F) > 160 * 1024 - 256 || F > 2 * COMB_TILE_W;
    const size_t comb_lds = tiled ? (size_t)COMB_TILE_W * 4 + (size_t)COMB_XS * 4 : comb_lds_bytes(F);

    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return I6FBW_ERR_INVALID_ARGUMENT;
    Pipeline& P = g_pipe[dev];
    std::lock_guard<std::mutex> lock(P.mu);
    { int rc = static_call ? device_init(P) : pipeline_init(P); if (rc != I6FBW_OK) return rc; }
    if (static_call) workspace = P.static_ws;

    hipStream_t s = (hipStream_t)stream_;
    char* ws = (char*)workspace;
    SeqMeta* meta = (SeqMeta*)(ws + l.meta);
    int* sync = (int*)(ws + l.sync);
    // More recursion workgroups than compute units: the instance of which two fit on a unit -- unless
    // the sequences can be longer than 4096 frames, which only the other instances run in double
    // precision (recurse_workgroup), or the automata are too large for one state per thread there (with
    // several states per thread and double vectors under its register cap it takes 1.5-1.8 us per frame
    // where the other instances take 0.5: two rounds of those are faster).
    const bool dense = 2 * B > P.n_cu && T <= 4096 && (long long)n_states <= (long long)REC_THREADS_DENSE * B;
    const bool big = !dense && (long long)n_states > (long long)BIG_STATES * B;
    // Small problems run stage after stage on the caller's stream; large ones overlap the stages.
    const int forced = static_call ? 0 : g_overlap_mode.load();
    // By default only where it pays (measured at F = 12001 unless said otherwise, ms per call stage
    // after stage / overlapped): a large dense tensor; a batch whose recursion workgroups leave half of
    // the compute units alone (T=400 B=100 F=5001: 0.33 / 0.36; T=200 B=256 F=5001: 0.34 / 0.43; with
    // up to 64 sequences T=600 B=32: 0.37 / 0.33, T=1000 B=32: 0.62 / 0.52, T=2000 B=16 F=3000: 1.39 /
    // 1.07); not with few frames (there is little recursion to hide: T=200 B=64 0.20 / 0.23, T=300 B=32
    // 0.19 / 0.20) nor, unless the sequences are long, with a handful of sequences (T=1000 B=8: 0.36 /
    // 0.34, T=4000 B=8 with large automata: 3.27 / 2.81).
    bool overlap = forced >= 0 ? forced != 0
                               : ((long long)T * B * F >= (1LL << 26) && 2 * B <= P.n_cu / 2 && T >= 384 && (B >= 12 || T >= 1000));
    // All 2B recursion workgroups must be on the machine at the same time (at most two per compute
    // unit): gather and dense write wait for their progress while occupying wave slots themselves.
    if (2 * B > (dense ? 2 : 1) * P.n_cu) overlap = false;
    // (a workgroup of the instance for large automata fills the register file of its compute unit: the kernels it
    // waits for need units of their own -- with 240 such workgroups on 256 units a forced overlap ran into the bound
    // of its waits)
    if (big && 2 * B > P.n_cu / 2) overlap = false;
    // Two workgroups of the dense instance are four waves per SIMD: beyond 104 registers each they
    // leave no room for the gather's waves, which they wait for.  (The compiler is asked for 96; how
    // close it gets depends on its version.)
    if (dense && P.dense_regs > 104) overlap = false;
    if (overlap) {
        // under stream capture: one stream, no in-memory waits between kernels, no synchronisation
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) overlap = false;
    }
    if (overlap) { int rc = runs_beside(P, s, &overlap); if (rc != I6FBW_OK) return rc; }
    hipStream_t sP = overlap ? P.sP : s, sR = overlap ? P.sR : s;
    const bool timed = g_prof.on && !static_call;     // stage timers create events
    if (timed) { std::lock_guard<std::mutex> plock(g_mutex); g_prof.n_calls++; }

    const dim3 g_grid((unsigned)B * ((T + TG - 1) / TG)), c_grid((unsigned)B * ((T + TC - 1) / TC));
    const dim3 p_grid(B, (T + TC - 1) / TC);
    const bool neglog = out_mode == I6FBW_OUT_NEG_LOG;      // the dense write then sums in log space (its NEGLOG instances)
    if ((long long)B * ((T + TG - 1) / TG) > 0x7fffffffLL) return I6FBW_ERR_INVALID_ARGUMENT;
    PrepArgs pa;
    pa.edges = edges; pa.edge_stride = edge_row_stride; pa.weights = weights;
    pa.start_end = start_end; pa.se_stride = se_row_stride; pa.seq_lens = seq_lens;
    pa.T = T; pa.B = B; pa.F = F; pa.E = E; pa.n_states = n_states; pa.best_path = 0; pa.count_wgs = overlap ? 1 : 0; pa.no_band = (input_flags & I6FBW_IN_ALL_FRAMES) ? 1 : 0; pa.dense = dense ? 1 : 0; pa.force_generic = f_too_large ? 1 : 0;
    pa.meta = meta; pa.sync = sync; pa.sortflag = (int*)(ws + l.sortflag); pa.seqbegin = (int*)(ws + l.seqbegin); pa.eidx = (int*)(ws + l.eidx); pa.renum = (int2*)(ws + l.renum);
    pa.ellA = (uint2*)(ws + l.ellA); pa.ellB = (uint2*)(ws + l.ellB);
    pa.crec = (uint4*)(ws + l.crec); pa.cbegin = (int*)(ws + l.cbegin); pa.demis = (int*)(ws + l.demis); pa.tband = (int2*)(ws + l.tband);
    pa.cflag = (int*)(ws + l.cflag); pa.wpfx = l.wpfx_stride > 0 ? (int*)(ws + l.wpfx) : nullptr; pa.wpfx_stride = l.wpfx_stride;
    GatherArgs ga;
    ga.am = am; ga.st_t = am_stride_t; ga.st_b = am_stride_b; ga.T = T; ga.B = B;
    ga.meta = meta; ga.demis = pa.demis; ga.tband = pa.tband; ga.gtab = (float*)(ws + l.gtab); ga.sync = sync;
    ga.scale = (input_flags & I6FBW_IN_LOG_PROBS) ? -LOG2E : LOG2E; ga.ascending = 0;
    GenArgs gen;
    gen.am = am; gen.st_t = am_stride_t; gen.st_b = am_stride_b; gen.sign = (input_flags & I6FBW_IN_LOG_PROBS) ? -1.f : 1.f;
    gen.edges = edges; gen.edge_stride = edge_row_stride; gen.weights = weights; gen.eidx = pa.eidx; gen.renum = pa.renum;
    gen.all_frames = (input_flags & I6FBW_IN_ALL_FRAMES) ? 1 : 0;
    RecArgs ra;
    ra.gen = gen;
    ra.T = T; ra.B = B; ra.prep_wgs = 3 * B; ra.meta = meta; ra.ellA = pa.ellA; ra.ellB = pa.ellB; ra.gtab = ga.gtab; ra.gtab_rw = ga.gtab;
    ra.alpha = (float*)(ws + l.alpha); ra.beta = (float*)(ws + l.beta);
    ra.offA = (double*)(ws + l.offA); ra.offB = (double*)(ws + l.offB); ra.sync = sync;
    CombArgs ca;
    ca.gen = gen;
    ca.T = T; ca.B = B; ca.F = F; ca.out_mode = out_mode;
    ca.meta = meta; ca.crec = pa.crec; ca.cbegin = pa.cbegin; ca.demis = pa.demis;
    ca.alpha = ra.alpha; ca.beta = ra.beta; ca.gtab = ga.gtab; ca.offA = ra.offA; ca.offB = ra.offB;
    ca.out = out; ca.sum_output = sum_output; ca.ost_t = out_stride_t; ca.ost_b = out_stride_b; ca.sync = sync;
    ca.tile_w = tiled ? COMB_TILE_W : 0;
    ca.direct_only = 0;
    // The dense tensor goes out in flat spans (fbw_flat) if it is one contiguous block in either
    // order of frames and sequences, rows are long enough for a span to cut at most two of them,
    // and the tensor is large (for small problems the row writer is as good).
    int flat_layout = -1;
    if (out_stride_b == (int64_t)F && out_stride_t == (int64_t)B * F) flat_layout = 0;
    else if (out_stride_t == (int64_t)F && out_stride_b == (int64_t)T * F) flat_layout = 1;
    const int writer = g_writer_mode.load();
    bool flat = (writer > 0 || (writer < 0 && (overlap || (long long)T * B * F >= (1LL << 26)))) && flat_layout >= 0 &&
                F >= FLAT_MIN_F && l.wpfx_stride > 0;
    FlatArgs fa;
    long long flat_grid = 0;
    if (flat) {
        const long long n = (T + TC - 1) / TC, rows = flat_layout == 0 ? B : 1;
        fa.c = ca; fa.layout = flat_layout;
        fa.K = FLAT_KMAX;
        fa.nW = (int)(((long long)TC * rows * F + 31 + (long long)fa.K * FLAT_W - 1) / ((long long)fa.K * FLAT_W));
        fa.shift = row_misalign_host(out);
        fa.cflag = (int*)(ws + l.cflag); fa.wpfx = (const int*)(ws + l.wpfx); fa.wpfx_stride = l.wpfx_stride;
        fa.cp = ga.gtab;
        fa.ahead = overlap ? FLAT_AHEAD : FLAT_AHEAD_ALONE;
        flat_grid = (long long)fa.ahead * B * (TC / FLAT_TCF) + (flat_layout == 0 ? n : n * B) * (fa.nW + rows * (TC / FLAT_TCF));
        if (flat_grid > 0x7fffffffLL || (long long)TC * rows * F >= (1LL << 31) - FLAT_W) flat = false;
    }
    ca.direct_only = flat ? 1 : 0;
    g_last_writer = flat ? 1 : 0;

    {
        // the scan also clears the header of the hand-off area, so it runs even without edges
        StageTimer tm(0, s, timed);
        hipLaunchKernelGGL(fbw_scan_sorted, dim3(std::max(1, (E + SCAN_BLOCK - 1) / SCAN_BLOCK)), dim3(256), 0, s,
                           E > 0 ? edges + 3 * edge_row_stride : nullptr, E, B, pa.sortflag, pa.seqbegin, sync);
        HIP_TRY(hipGetLastError());
    }
    // Where the recursion kernel is started: beside the preparation if its 2B workgroups leave at
    // least half of the compute units empty (the preparation's workgroups need most of a unit's
    // LDS and could otherwise find no room while the recursion waits for them), else behind it.
    const bool early = overlap && 2 * B <= P.n_cu / 2;
    // The preparation's workgroups can do the gate's wait themselves (one kernel less in front of the gather)
    // where they cannot be in the recursion's way: a preparation workgroup and a recursion workgroup do not
    // share a compute unit, the order in which the two kernels are placed is not ours, and a preparation
    // workgroup that waits keeps its unit -- so only if both grids fit with a unit per workgroup.  Workgroups are
    // dealt out to the device's XCDs in turn, so the units have to be there XCD by XCD, each with its share of either
    // grid rounded up: 51 sequences are 20 + 13 workgroups for the first XCD's 32 units -- 5 B <= 256, and the
    // thirteenth recursion workgroup waited for a unit until the preparation's waits ran out.  (Four units per XCD
    // are left over for whatever else is on the machine.)
    constexpr int XCDS = 8;
    const bool gate_in_prepare = early && (3 * B + XCDS - 1) / XCDS + (2 * B + XCDS - 1) / XCDS <= P.n_cu / XCDS - 4;
    pa.gate_need = gate_in_prepare ? 2 * B : 0;
    auto launch_recursion = [&]() -> int {
        { StageTimer tm(2, sR, timed); if (dense) hipLaunchKernelGGL(fbw_recurse_dense<true>, dim3(2 * B), dim3(REC_BLOCK_DENSE), sizeof(float) * REC_LDS_FLOATS_F32, sR, ra);
          else if (big) hipLaunchKernelGGL(fbw_recurse_big<true>, dim3(2 * B), dim3(REC_BLOCK_BIG), 0, sR, ra);
          else if (early) hipLaunchKernelGGL((fbw_recurse<true, true>), dim3(2 * B), dim3(REC_BLOCK), 0, sR, ra);
          else hipLaunchKernelGGL((fbw_recurse<true, false>), dim3(2 * B), dim3(REC_BLOCK), 0, sR, ra); }
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipEventRecord(P.doneR, sR));
        return I6FBW_OK;
    };
    // Whatever way this function is left once the library streams have been given work: the caller's
    // stream waits for them, so that nothing enqueued on it afterwards (the release of a torch-owned
    // workspace, say) can overtake kernels that still use the workspace.
    struct JoinGuard {
        Pipeline& P; hipStream_t s; bool armed = false, joined = false;
        ~JoinGuard() {
            if (!armed || joined) return;
            if (hipEventRecord(P.doneP, P.sP) == hipSuccess) (void)hipStreamWaitEvent(s, P.doneP, 0);
            if (hipEventRecord(P.doneR, P.sR) == hipSuccess) (void)hipStreamWaitEvent(s, P.doneR, 0);
        }
    } join_guard{P, s};
    if (overlap) {
        join_guard.armed = true;
        // The library streams are released when the scan is done, i.e. while the preparation's
        // workgroups are being placed.  The recursion's 2B large workgroups need nine free wave
        // slots on one compute unit each and find them while the machine is still almost empty;
        // they wait in memory for the preparation to finish (fbw_prepare counts its workgroups),
        // and their loader waves later for the gather's strip flags.
        HIP_TRY(hipEventRecord(P.start, s));
        HIP_TRY(hipStreamWaitEvent(sP, P.start, 0));
        if (early) {
            HIP_TRY(hipStreamWaitEvent(sR, P.start, 0));
            int rc = launch_recursion(); if (rc != I6FBW_OK) return rc;
        }
    }
    {
        StageTimer tm(0, s, timed);
        launch_prepare(P, pa, s);
        HIP_TRY(hipGetLastError());
    }
    if (overlap && !early) {
        HIP_TRY(hipEventRecord(P.fork, s));
        HIP_TRY(hipStreamWaitEvent(sR, P.fork, 0));
        int rc = launch_recursion(); if (rc != I6FBW_OK) return rc;
    }
    // (with the flat writer, the row writer for the sequences fbw_flat leaves out is started below, behind the gather)
    ca.pad_rows = (!flat && !overlap) ? 1 : 0;
    if (!flat && overlap) {
        // Rows of frames beyond seq_len depend on seq_lens only: written beside the preparation, which
        // leaves the memory system idle.  (Stage after stage the row writer takes them, see pad_rows.)
        StageTimer tm(4, sP, timed);
        hipLaunchKernelGGL(fbw_padfill, p_grid, dim3(COMB_THREADS), 0, sP, seq_lens, T, B, F, out_mode, out, (long long)out_stride_t,
                           (long long)out_stride_b, sum_output);
        HIP_TRY(hipGetLastError());
    }
    if (overlap) HIP_TRY(hipEventRecord(P.doneP, sP));

    if (!overlap) {
        { StageTimer tm(1, s, timed); hipLaunchKernelGGL(fbw_gather<false>, g_grid, dim3(256), 0, s, ga); }
        HIP_TRY(hipGetLastError());
        { StageTimer tm(2, s, timed); if (dense) hipLaunchKernelGGL(fbw_recurse_dense<false>, dim3(2 * B), dim3(REC_BLOCK_DENSE), sizeof(float) * REC_LDS_FLOATS_F32, s, ra);
          else if (big) hipLaunchKernelGGL(fbw_recurse_big<false>, dim3(2 * B), dim3(REC_BLOCK_BIG), 0, s, ra);
          else hipLaunchKernelGGL(fbw_recurse<false>, dim3(2 * B), dim3(REC_BLOCK), 0, s, ra); }
        HIP_TRY(hipGetLastError());
        if (flat) {
            // (the row kernel first: it only has the sequences that are too large for the other one)
            { StageTimer tm(4, s, timed); launch_combine<false>(neglog, c_grid, comb_lds, s, ca); }
            { StageTimer tm(3, s, timed); launch_flat<false>(neglog, dim3((unsigned)flat_grid), s, fa); }
        } else { StageTimer tm(3, s, timed); launch_combine<false>(neglog, c_grid, comb_lds, s, ca); }
        HIP_TRY(hipGetLastError());
        return I6FBW_OK;
    }

    // A running grid of small workgroups refills every wave slot it frees, so gather and dense
    // write (which also wait for recursion progress while they occupy LDS and wave slots) are
    // held back until every recursion workgroup is on the machine -- normally long since.
    // (Or by the preparation's workgroups at their end, see gate_in_prepare.)
    if (!gate_in_prepare) {
        hipLaunchKernelGGL(fbw_gate, dim3(1), dim3(64), 0, s, sync, 2 * B);
        HIP_TRY(hipGetLastError());
    }
    { StageTimer tm(1, s, timed); hipLaunchKernelGGL(fbw_gather<true>, g_grid, dim3(256), 0, s, ga); }
    HIP_TRY(hipGetLastError());
    if (flat) {
        // fbw_flat writes every row except those of sequences too large for its posterior jobs: these go
        // row by row through fbw_combine on the second library stream, beside fbw_flat (the two kernels
        // do not wait for each other).  It is started behind the gather like fbw_flat itself: its
        // workgroups wait for the gather's strips while they hold registers and wave slots, so they
        // must not be on the machine before the gather's own are (three of them fill a compute unit's
        // register file).  It has nothing to do for the usual batch.
        HIP_TRY(hipEventRecord(P.gathered, s));
        HIP_TRY(hipStreamWaitEvent(sP, P.gathered, 0));
        { StageTimer tm(4, sP, timed); launch_combine<true>(neglog, c_grid, comb_lds, sP, ca); }
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipEventRecord(P.doneP, sP));
    }
    // The dense write follows the gather on the same stream (its workgroups would only take wave
    // slots away from the gather before that: by then the two recursions are about to meet in the
    // middle of the sequences, where the dense write begins); each of its workgroups waits for the
    // recursion progress it needs.
#ifdef I6_TRACE
    if (getenv("I6FBW_DBG_SERIAL_COMBINE")) HIP_TRY(hipStreamWaitEvent(s, P.doneR, 0));
#endif
    if (flat) { StageTimer tm(3, s, timed); launch_flat<true>(neglog, dim3((unsigned)flat_grid), s, fa); }
    else { StageTimer tm(3, s, timed); launch_combine<true>(neglog, c_grid, comb_lds, s, ca); }
    HIP_TRY(hipGetLastError());
    // join: both finish well before the dense write does
    HIP_TRY(hipStreamWaitEvent(s, P.doneP, 0));
    HIP_TRY(hipStreamWaitEvent(s, P.doneR, 0));
    join_guard.joined = true;
    return I6FBW_OK;
}
}  // namespace

extern "C" {

// a stream that is being captured into a graph can neither be waited for nor carry the events of
// the status ring: no report from there
static bool is_capturing(hipStream_t s) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone;
}

int i6fbw_read_status(const void* workspace, int B, void* stream, int* code, int* seq) {
    if (!workspace || B <= 0 || !code || !seq) return I6FBW_ERR_INVALID_ARGUMENT;
    if (is_capturing((hipStream_t)stream)) { *code = I6FBW_OK; *seq = -1; return I6FBW_OK; }
    // the meta records sit at the start of the workspace, the abort flag of the hand-off area right
    // behind them: one copy brings both
    const size_t flag_at = align256(sizeof(SeqMeta) * (size_t)B);
    char* host = (char*)malloc(flag_at + sizeof(int));
    if (!host) return I6FBW_ERR_INVALID_ARGUMENT;
    hipError_t e = hipMemcpyAsync(host, workspace, flag_at + sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) { g_last_hip_error = e; free(host); return I6FBW_ERR_LAUNCH; }
    int aborted = 0;
    memcpy(&aborted, host + flag_at, sizeof(int));
    const SeqMeta* meta = (const SeqMeta*)host;
    *code = aborted ? I6FBW_ERR_TIMEOUT : I6FBW_OK; *seq = -1;
    if (aborted) forget_stream_checks();
    for (int b = 0; b < B; b++) {
        // positive values mark sequences that took the general path
        const int c = meta[b].err < 0 ? meta[b].err : (meta[b].errA < 0 ? meta[b].errA : (meta[b].errB < 0 ? meta[b].errB : 0));
        if (c) { *code = c; *seq = b; break; }
    }
    free(host);
    return I6FBW_OK;
}

int i6fbw_post_status(void* workspace, int B, void* stream) {
    if (!workspace || B <= 0) return I6FBW_ERR_INVALID_ARGUMENT;
    if (is_capturing((hipStream_t)stream)) return I6FBW_OK;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return I6FBW_ERR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> lock(g_pipe[dev].mu);
    StatusRing& r = g_status[dev];
    if (!r.host) HIP_TRY(hipHostMalloc((void**)&r.host, sizeof(int) * 2 * StatusRing::SLOTS, hipHostMallocDefault));
    const int i = r.next;
    r.next = (r.next + 1) % StatusRing::SLOTS;
    status_collect(r, i, true);                  // the oldest report, if the ring has come round to it
    if (!r.ev[i]) HIP_TRY(hipEventCreateWithFlags(&r.ev[i], hipEventDisableTiming));
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    // {code, seq} go through two unused ints of the hand-off header, which sits behind the meta records
    int* sync = (int*)(ws + align256(sizeof(SeqMeta) * (size_t)B));
    hipLaunchKernelGGL(fbw_status_reduce, dim3(1), dim3(256), 0, s, (const SeqMeta*)ws, B, sync, sync + 4);
    HIP_TRY(hipGetLastError());
    r.host[2 * i] = I6FBW_OK; r.host[2 * i + 1] = -1;
    HIP_TRY(hipMemcpyAsync(r.host + 2 * i, sync + 4, 2 * sizeof(int), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipEventRecord(r.ev[i], s));
    r.used[i] = true;
    return I6FBW_OK;
}

int i6fbw_poll_status(int wait, int* code, int* seq) {
    if (!code || !seq) return I6FBW_ERR_INVALID_ARGUMENT;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return I6FBW_ERR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> lock(g_pipe[dev].mu);
    StatusRing& r = g_status[dev];
    // oldest first; reports arrive in the order of the calls (on one stream), so the first one that
    // is still on its way ends the search: a poll costs one or two event queries, not sixty-four
    for (int k = 0; k < StatusRing::SLOTS; k++)
        if (!status_collect(r, (r.next + k) % StatusRing::SLOTS, wait != 0)) break;
    *code = r.held_code; *seq = r.held_seq;
    r.held_code = I6FBW_OK; r.held_seq = -1;
    if (*code == I6FBW_ERR_TIMEOUT) g_pipe[dev].checked.clear();      // (this device's lock is held)
    return I6FBW_OK;
}

void i6fbw_set_status_mode(int mode) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_status_mode = mode <= 0 ? 0 : (mode == 1 ? 1 : 2);
}

int i6fbw_get_status_mode(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    return g_status_mode;
}

const char* i6fbw_strerror(int code) {
    switch (code) {
        case I6FBW_OK: return "ok";
        case I6FBW_ERR_INVALID_ARGUMENT: return "invalid argument";
        case I6FBW_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
        case I6FBW_ERR_LAUNCH: return "HIP call failed";
        case I6FBW_ERR_SEQ_TOO_LARGE: return "best path: a sequence on the general path does not fit its share of the workspace";
        case I6FBW_ERR_BAD_INDEX: return "sequence, emission or state index out of range";
        case I6FBW_ERR_TIMEOUT: return "a kernel gave up waiting for another stage of the same call";
        case I6FBW_ERR_STATIC_WORKSPACE: return "the problem needs more workspace than the built-in buffer of i6fbw_run_static holds (32 MiB)";
        default: return "unknown status";
    }
}

int i6fbw_set_spin_limit(int polls) {
    const int v = polls > 0 ? polls : SPIN_LIMIT;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return I6FBW_ERR_INVALID_ARGUMENT;
    // no call of the library is being enqueued on this device while the limit changes, and none that was enqueued
    // before is still running: a kernel sees one limit from start to end
    std::lock_guard<std::mutex> lock(g_pipe[dev].mu);
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(g_spin_limit), &v, sizeof(int)));
    return I6FBW_OK;
}

void i6fbw_set_dense_writer(int mode) { g_writer_mode = mode < 0 ? -1 : (mode ? 1 : 0); }
int i6fbw_last_dense_writer(void) { return g_last_writer.load(); }

void i6fbw_set_band(int on) { g_all_frames_default = on ? 0 : I6FBW_IN_ALL_FRAMES; }

void i6fbw_set_overlap(int mode) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_overlap_mode = mode < 0 ? -1 : (mode ? 1 : 0);
}

#ifdef I6_TRACE
int i6fbw_debug_trace(void* host, int n) { return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_trace), sizeof(unsigned long long) * n); }
int i6fbw_debug_trace_set(const void* host, int n) { return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_trace), host, sizeof(unsigned long long) * n); }
#endif

// Text dumps of fbw_op.cu:155-224.  Host code: device-to-host copies and file output.
int i6fbw_dump_alignment(const void* workspace, int T, int B, int E, const int32_t* start_end, int64_t se_row_stride,
                         float pruning, unsigned batch_idx, const char* directory, void* stream) {
    if (!workspace || !start_end || !directory || T <= 0 || B <= 0 || E < 0) return I6FBW_ERR_INVALID_ARGUMENT;
    const Layout l = make_layout(T, B, E);
    std::vector<SeqMeta> meta(B);
    std::vector<int32_t> se(2 * (size_t)B);
    hipStream_t s = (hipStream_t)stream;
    HIP_TRY(hipStreamSynchronize(s));
    HIP_TRY(hipMemcpy(meta.data(), (const char*)workspace + l.meta, sizeof(SeqMeta) * B, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(se.data(), start_end, sizeof(int32_t) * B, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(se.data() + B, start_end + se_row_stride, sizeof(int32_t) * B, hipMemcpyDeviceToHost));
    std::vector<float> rows;
    std::vector<double> rows64;
    std::vector<int2> renum;
    for (int b = 0; b < B; b++) {
        const std::string name = std::string(directory) + "/alignment.dump." + std::to_string(batch_idx) + "." + std::to_string(b);
        FILE* f = fopen(name.c_str(), "w");
        if (!f) return I6FBW_ERR_INVALID_ARGUMENT;
        const SeqMeta& m = meta[b];
        const bool ok = m.err >= 0 && m.errA >= 0 && m.errB >= 0;   // (a sequence with a reported problem has no rows)
        const bool general = ok && (m.err > 0 || m.errA > 0 || m.errB > 0);
        const long long first = se[b], last = se[B + b];           // the reference walks the ids start..end
        // frame 0 is written even for an empty sequence (fbw_op.cu:177); it holds the start state only
        const int frames = !ok ? 0 : (m.L > 0 && m.n_edges > 0 ? m.L : 1);
        const bool have_rows = ok && m.L > 0 && m.n_edges > 0;
        // a sequence on the general path keeps its rows in double where they fit, and in natural-log units
        const long long soff = state_off(m.edge_begin, b);
        const long long share = state_off((long long)m.edge_begin + m.n_edges, b + 1) - soff;
        const long long groom = (long long)T * (slot_off((long long)m.edge_begin + m.n_edges, b + 1) - slot_off(m.edge_begin, b)) / 2;
        const bool r64 = general && 2LL * m.SP <= share && groom >= 4LL * m.SP;
        const float unit = general ? 1.f : LN2;
        if (have_rows) {
            const char* src = (const char*)workspace + l.alpha + sizeof(float) * (size_t)T * soff;
            hipError_t e;
            if (r64) { rows64.resize((size_t)m.L * m.SP); e = hipMemcpy(rows64.data(), src, sizeof(double) * rows64.size(), hipMemcpyDeviceToHost); }
            else { rows.resize((size_t)m.L * m.SP); e = hipMemcpy(rows.data(), src, sizeof(float) * rows.size(), hipMemcpyDeviceToHost); }
            if (e != hipSuccess) { g_last_hip_error = e; fclose(f); return I6FBW_ERR_LAUNCH; }
            if (m.pad & 2) {
                // state ids spread over a wide range: their numbers within the sequence sit in an open-addressing table
                renum.resize(renum_capacity(m.n_edges));
                e = hipMemcpy(renum.data(), (const char*)workspace + l.renum + sizeof(int2) * 2 * (size_t)soff, sizeof(int2) * renum.size(),
                              hipMemcpyDeviceToHost);
                if (e != hipSuccess) { g_last_hip_error = e; fclose(f); return I6FBW_ERR_LAUNCH; }
            }
        }
        // number of state id sid within the sequence, -1 if the sequence does not name it
        auto local = [&](long long sid) -> long long {
            if (!(m.pad & 2)) { const long long loc = sid - m.state_min; return loc >= 0 && loc < m.S ? loc : -1; }
            const unsigned cap = (unsigned)renum.size();
            unsigned h = renum_home((int)sid, cap);
            while (true) {
                if (renum[h].x == (int)sid + 1) return renum[h].y;
                if (renum[h].x == 0) return -1;
                h = h + 1 == cap ? 0 : h + 1;
            }
        };
        for (int t = 0; t < frames; t++) {
            // value of state id s in natural-log units (rows of the fast kernels are stored in units of
            // log 2; all rows are relative to an offset that cancels in the normalisation)
            auto value = [&](long long sid) -> float {
                if (!have_rows) return sid == first ? 0.f : INFINITY;
                const long long loc = local(sid);
                if (loc < 0) return INFINITY;
                return r64 ? (float)rows64[(size_t)t * m.SP + loc] : rows[(size_t)t * m.SP + loc] * unit;
            };
            float sum = INFINITY;
            for (long long sid = first; sid <= last; sid++) {
                const float val = value(sid);
                const float diff = val - sum;
                if (!std::isnan(diff)) sum = -log1pf(expf(-fabsf(diff))) + fminf(sum, val);
            }
            for (long long sid = first; sid <= last; sid++) {
                const float val = value(sid) - sum;
                if (val <= pruning) fprintf(f, "%d %lld %g\n", t, sid - first, val);
            }
        }
        fclose(f);
    }
    return I6FBW_OK;
}

int i6fbw_dump_output(const float* out, int64_t out_stride_t, int64_t out_stride_b, const int32_t* seq_lens, int T, int B,
                      int F, float pruning, unsigned batch_idx, const char* directory, void* stream) {
    if (!out || !seq_lens || !directory || T <= 0 || B <= 0 || F <= 0) return I6FBW_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    HIP_TRY(hipStreamSynchronize(s));
    std::vector<int32_t> lens(B);
    HIP_TRY(hipMemcpy(lens.data(), seq_lens, sizeof(int32_t) * B, hipMemcpyDeviceToHost));
    std::vector<float> row(F);
    for (int b = 0; b < B; b++) {
        const std::string name = std::string(directory) + "/target.dump." + std::to_string(batch_idx) + "." + std::to_string(b);
        FILE* f = fopen(name.c_str(), "w");
        if (!f) return I6FBW_ERR_INVALID_ARGUMENT;
        for (int t = 0; t < T; t++) {
            if (t > 0 && (unsigned)t >= (unsigned)lens[b]) break;
            if (hipMemcpy(row.data(), out + (int64_t)t * out_stride_t + (int64_t)b * out_stride_b, sizeof(float) * F,
                          hipMemcpyDeviceToHost) != hipSuccess) { fclose(f); return I6FBW_ERR_LAUNCH; }
            for (int e = 0; e < F; e++)
                if (row[e] <= pruning) fprintf(f, "%d %d %g\n", t, e, row[e]);
        }
        fclose(f);
    }
    return I6FBW_OK;
}

const char* i6fbw_last_hip_error(void) { return g_last_hip_error == hipSuccess ? "" : hipGetErrorString(g_last_hip_error); }

void i6fbw_profile_enable(int on) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_prof.on = on != 0;
    g_prof.n_pairs = 0;
    g_prof.n_calls = 0;
}

int i6fbw_profile_read(float* stage_ms) {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (int st = 0; st < I6FBW_N_STAGES; st++) stage_ms[st] = 0.f;
    const int calls = g_prof.n_calls;
    if (calls == 0) return 0;
    for (int i = 0; i < g_prof.n_pairs; i++) {
        float ms = 0.f;
        if (hipEventSynchronize(g_prof.b[i]) != hipSuccess) continue;
        if (hipEventElapsedTime(&ms, g_prof.a[i], g_prof.b[i]) != hipSuccess) continue;
        stage_ms[g_prof.stage[i]] += ms / calls;
    }
    g_prof.n_pairs = 0;
    g_prof.n_calls = 0;
    return calls;
}

}  // extern "C"

#include "viterbi_kernels.inc"
#include "fsa_builders.inc"
