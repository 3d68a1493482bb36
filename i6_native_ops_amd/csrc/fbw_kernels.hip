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
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/i6fbw.h"

namespace {

constexpr int KMAX = 8;               // in-/out-degree held in registers by the recursion
constexpr int EB_MAX = 8192;          // edges of one sequence (capacity of the LDS sort)
constexpr int F_BITMAP_MAX = 131072;  // emission ids covered by the LDS presence bitmap
constexpr int S_MAX = 4096;           // states of one sequence (largest recursion class)
constexpr int D_MAX = 4096;           // distinct emissions of one sequence
constexpr int TG = 8;                 // frames per gather workgroup
constexpr int TC = 8;                 // frames per combine workgroup
constexpr int RENORM = 8;             // frames between renormalisations of the state vector
constexpr int COMB_THREADS = 256;
constexpr int COMB_JD = D_MAX / COMB_THREADS;
constexpr unsigned NO_STATE = 0xFFFFu;
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
    int pad;
};

__host__ __device__ inline long long round16(long long x) { return (x + 15) & ~15LL; }
// Workspace offsets of a sequence follow from the number of edges before it, so that no
// prefix sum over sequences (and no cross-workgroup dependency) is needed.
__host__ __device__ inline long long state_off(long long edge_begin, int b) { return round16(2 * edge_begin) + 32LL * b; }
__host__ __device__ inline long long slot_off(long long edge_begin, int b) { return round16(edge_begin) + 32LL * b; }

struct Layout {
    size_t meta, ellA, ellB, crec, cbegin, demis, offA, offB, alpha, beta, gtab, total;
    long long ss_total, gg_total;
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

Layout make_layout(long long T, long long B, long long E) {
    Layout l;
    l.ss_total = round16(2 * E) + 32 * B + 16;
    l.gg_total = round16(E) + 32 * B + 16;
    size_t o = 0;
    l.meta = o;   o = align256(o + sizeof(SeqMeta) * B);
    l.ellA = o;   o = align256(o + sizeof(uint2) * KMAX * l.ss_total);
    l.ellB = o;   o = align256(o + sizeof(uint2) * KMAX * l.ss_total);
    l.crec = o;   o = align256(o + sizeof(uint4) * (E + 1));
    l.cbegin = o; o = align256(o + sizeof(int) * l.gg_total);
    l.demis = o;  o = align256(o + sizeof(int) * l.gg_total);
    l.offA = o;   o = align256(o + sizeof(double) * B * T);
    l.offB = o;   o = align256(o + sizeof(double) * B * T);
    l.alpha = o;  o = align256(o + sizeof(float) * l.ss_total * T);
    l.beta = o;   o = align256(o + sizeof(float) * l.ss_total * T);
    l.gtab = o;   o = align256(o + sizeof(float) * l.gg_total * T);
    l.total = o;
    return l;
}

// ---------------------------------------------------------------------------------------------
// small device helpers
// ---------------------------------------------------------------------------------------------
__device__ inline int seq_error(const SeqMeta& m) { return m.err ? m.err : (m.errA ? m.errA : m.errB); }

// Recursion class of a sequence: 0 nothing to do, 1..3 by size, -1 error.
__device__ inline int rec_class(const SeqMeta& m) {
    if (seq_error(m)) return -1;
    if (m.L == 0 || m.n_edges == 0) return 0;
    if (m.SP <= 512 && m.DP <= 512) return 1;
    if (m.SP <= 2048 && m.DP <= 2048) return 2;
    return 3;
}
// Combine class: 1 handles errors, empty sequences and sequences of up to 1024 edges.
__device__ inline int comb_class(const SeqMeta& m) {
    if (seq_error(m) || m.L == 0 || m.n_edges == 0) return 1;
    return m.n_edges <= 1024 ? 1 : 2;
}

__device__ inline float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
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
    SeqMeta* meta; uint2* ellA; uint2* ellB; uint4* crec; int* cbegin; int* demis;
};

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

// first index i in [0,n) with (keys[i] >> 32) >= p
__device__ inline int lower_bound_hi(const unsigned long long* keys, int n, unsigned p) {
    int lo = 0, hi = n;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if ((unsigned)(keys[mid] >> 32) < p) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// grid (3, B): role 0 orders the edges of sequence b by target state (alpha), role 1 by source
// state (beta), role 2 by emission slot (combine) and writes the shared part of the meta record.
__global__ __launch_bounds__(1024) void fbw_prepare(PrepArgs a) {
    __shared__ unsigned long long keys[EB_MAX];
    __shared__ int eidx[EB_MAX];
    __shared__ unsigned bitmap[F_BITMAP_MAX / 32];
    __shared__ int wordpfx[F_BITMAP_MAX / 32];
    __shared__ int wsum[16];
    __shared__ int s_lt, s_bad, s_kmax;
    __shared__ unsigned s_min, s_max;

    const int role = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int32_t* e_from = a.edges;
    const int32_t* e_to = a.edges + a.edge_stride;
    const int32_t* e_emis = a.edges + 2 * a.edge_stride;
    const int32_t* e_seq = a.edges + 3 * a.edge_stride;
    const int E = a.E;

    if (tid == 0) { s_lt = 0; s_bad = 0; s_kmax = 0; s_min = 0xffffffffu; s_max = 0u; }
    __syncthreads();

    // pass 1: count the edges of earlier sequences and of this one, state range, index checks
    const int chunk = (E + 1023) / 1024;
    const int lo = min(E, tid * chunk), hi = min(E, lo + chunk);
    int lt = 0, eq = 0, bad = 0;
    unsigned mn = 0xffffffffu, mx = 0u;
    for (int i = lo; i < hi; i++) {
        unsigned s = (unsigned)e_seq[i];
        lt += s < (unsigned)b;
        if (s == (unsigned)b) {
            eq++;
            unsigned f = (unsigned)e_from[i], t = (unsigned)e_to[i];
            mn = min(mn, min(f, t)); mx = max(mx, max(f, t));
            if (f >= (unsigned)a.n_states || t >= (unsigned)a.n_states || (unsigned)e_emis[i] >= (unsigned)a.F) bad = 1;
        }
        if (b == 0 && s >= (unsigned)a.B) bad = 1;
    }
    if (lt) atomicAdd(&s_lt, lt);
    if (bad) atomicOr(&s_bad, 1);
    if (eq) { atomicMin(&s_min, mn); atomicMax(&s_max, mx); }
    int n_edges;
    int pos = block_excl_scan(eq, wsum, 16, &n_edges);   // barriers inside publish the atomics too
    const int edge_begin = s_lt;

    const unsigned st_state = (unsigned)a.start_end[b], en_state = (unsigned)a.start_end[a.se_stride + b];
    unsigned smin = min(min(s_min, st_state), en_state), smax = max(max(s_max, st_state), en_state);
    int err = 0;
    if (s_bad || st_state >= (unsigned)a.n_states || en_state >= (unsigned)a.n_states) err = I6FBW_ERR_BAD_INDEX;
    else if (n_edges > EB_MAX) err = I6FBW_ERR_SEQ_TOO_MANY_EDGES;
    const unsigned sl = (unsigned)a.seq_lens[b];
    const int L = (sl >= 1u && sl <= (unsigned)a.T) ? (int)sl : 0;
    long long S = (long long)smax - smin + 1;
    if (!err && n_edges > 0 && S > 2LL * n_edges + 2) err = I6FBW_ERR_SEQ_SPARSE_STATES;
    if (n_edges == 0) S = 1;
    if (!err && S > S_MAX) err = I6FBW_ERR_SEQ_TOO_LARGE;
    const int SP = (int)round16(S);
    const long long soff = state_off(edge_begin, b), goff = slot_off(edge_begin, b);

    int D = 0;
    if (!err && n_edges > 0) {
        // pass 2: stable list of this sequence's edge indices
        for (int i = lo; i < hi; i++)
            if ((unsigned)e_seq[i] == (unsigned)b) eidx[pos++] = i;
        // emission presence bitmap -> slot = rank of the emission id among the distinct ones
        const int nwords = (a.F + 31) >> 5;
        for (int w = tid; w < nwords; w += 1024) bitmap[w] = 0u;
        __syncthreads();
        for (int i = tid; i < n_edges; i += 1024) {
            unsigned em = (unsigned)e_emis[eidx[i]];
            atomicOr(&bitmap[em >> 5], 1u << (em & 31));
        }
        __syncthreads();
        const int wpt = (nwords + 1023) / 1024;
        const int w0 = min(nwords, tid * wpt), w1 = min(nwords, w0 + wpt);
        int c = 0;
        for (int w = w0; w < w1; w++) c += __popc(bitmap[w]);
        int run = block_excl_scan(c, wsum, 16, &D);
        for (int w = w0; w < w1; w++) { wordpfx[w] = run; run += __popc(bitmap[w]); }
        __syncthreads();
        if (D > D_MAX) err = I6FBW_ERR_SEQ_TOO_LARGE;
    }
    const int DP = (int)round16(D > 0 ? D : 1);

    if (role == 2 && tid == 0) {
        SeqMeta* m = a.meta + b;
        m->edge_begin = edge_begin; m->n_edges = n_edges; m->state_min = (int)smin;
        m->S = (int)S; m->SP = SP; m->D = D; m->DP = DP; m->L = L;
        m->start_local = (int)(st_state - smin); m->end_local = (int)(en_state - smin);
        m->err = err; m->pad = 0;
    }
    if (err || n_edges == 0) {
        if (tid == 0) {
            if (role == 0) { a.meta[b].Kin = 0; a.meta[b].errA = 0; }
            if (role == 1) { a.meta[b].Kout = 0; a.meta[b].errB = 0; }
        }
        return;
    }

    auto slot_of = [&](unsigned em) -> unsigned {
        return (unsigned)wordpfx[em >> 5] + (unsigned)__popc(bitmap[em >> 5] & ((1u << (em & 31)) - 1u));
    };

    // sort keys: (primary << 32) | stable position; ties keep the input order
    int N = 2;
    while (N < n_edges) N <<= 1;
    for (int i = tid; i < N; i += 1024) {
        unsigned long long k = ~0ull;
        if (i < n_edges) {
            int e = eidx[i];
            unsigned p = role == 0 ? (unsigned)e_to[e] - smin : role == 1 ? (unsigned)e_from[e] - smin : slot_of((unsigned)e_emis[e]);
            k = ((unsigned long long)p << 32) | (unsigned)i;
        }
        keys[i] = k;
    }
    __syncthreads();
    for (int k = 2; k <= N; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < N; i += 1024) {
                int ixj = i ^ j;
                if (ixj > i) {
                    unsigned long long x = keys[i], y = keys[ixj];
                    bool up = (i & k) == 0;
                    if ((x > y) == up) { keys[i] = y; keys[ixj] = x; }
                }
            }
            __syncthreads();
        }
    }

    if (role < 2) {
        // ELL table: entry (k, s) = k-th edge (in input order) entering (role 0) / leaving (role 1)
        // local state s, as {other state | slot << 16, weight}; unused entries point at NO_STATE.
        uint2* ell = (role == 0 ? a.ellA : a.ellB) + (size_t)KMAX * soff;
        int kmax = 0;
        for (int i = tid; i < n_edges; i += 1024) {
            unsigned p = (unsigned)(keys[i] >> 32);
            kmax = max(kmax, i - lower_bound_hi(keys, n_edges, p) + 1);
        }
        if (kmax) atomicMax(&s_kmax, kmax);
        __syncthreads();
        const int K = s_kmax;
        const int kerr = K > KMAX ? I6FBW_ERR_SEQ_DEGREE : 0;
        if (tid == 0) {
            if (role == 0) { a.meta[b].Kin = K; a.meta[b].errA = kerr; }
            else { a.meta[b].Kout = K; a.meta[b].errB = kerr; }
        }
        if (kerr) return;
        for (int i = tid; i < K * SP; i += 1024) ell[i] = make_uint2(NO_STATE, 0u);
        __syncthreads();
        for (int i = tid; i < n_edges; i += 1024) {
            unsigned p = (unsigned)(keys[i] >> 32);
            int k = i - lower_bound_hi(keys, n_edges, p);
            int e = eidx[(unsigned)keys[i]];
            unsigned other = (role == 0 ? (unsigned)e_from[e] : (unsigned)e_to[e]) - smin;
            unsigned slot = slot_of((unsigned)e_emis[e]);
            ell[(size_t)k * SP + p] = make_uint2(other | (slot << 16), __float_as_uint(a.weights[e]));
        }
    } else {
        // combine order: edges sorted by slot; CSR begin per slot; list of distinct emission ids
        uint4* crec = a.crec + edge_begin;
        for (int i = tid; i < n_edges; i += 1024) {
            int e = eidx[(unsigned)keys[i]];
            unsigned f = (unsigned)e_from[e] - smin, t = (unsigned)e_to[e] - smin;
            crec[i] = make_uint4(f | (t << 16), __float_as_uint(a.weights[e]), (unsigned)(keys[i] >> 32), 0u);
        }
        int* cb = a.cbegin + goff;
        for (int d = tid; d <= D; d += 1024) cb[d] = d == D ? n_edges : lower_bound_hi(keys, n_edges, (unsigned)d);
        int* de = a.demis + goff;
        const int nwords = (a.F + 31) >> 5;
        for (int w = tid; w < nwords; w += 1024) {
            unsigned bits = bitmap[w];
            int r = wordpfx[w];
            while (bits) {
                int bit = __ffs((int)bits) - 1;
                de[r++] = w * 32 + bit;
                bits &= bits - 1;
            }
        }
        for (int d = D + tid; d < DP; d += 1024) de[d] = 0;
    }
}

// ---------------------------------------------------------------------------------------------
// stage 2: gather  gtab[b][t][slot] = am[t, b, demis[b][slot]]  for t < L_b
// ---------------------------------------------------------------------------------------------
struct GatherArgs {
    const float* am; long long st_t, st_b;
    int T, B;
    const SeqMeta* meta; const int* demis; float* gtab;
};

__global__ __launch_bounds__(256) void fbw_gather(GatherArgs a) {
    const int b = blockIdx.y, t0 = blockIdx.x * TG;
    const SeqMeta m = a.meta[b];
    if (rec_class(m) <= 0 || t0 >= m.L) return;
    const long long goff = slot_off(m.edge_begin, b);
    const int* de = a.demis + goff;
    float* g = a.gtab + (size_t)a.T * goff;
    const float* am = a.am + (long long)b * a.st_b;
    const int nt = min(TG, m.L - t0);
    for (int idx = threadIdx.x; idx < m.DP; idx += 256) {
        const int e = de[idx];
        float v[TG];
#pragma unroll
        for (int tt = 0; tt < TG; tt++)
            if (tt < nt) v[tt] = am[(long long)(t0 + tt) * a.st_t + e];
#pragma unroll
        for (int tt = 0; tt < TG; tt++)
            if (tt < nt) g[(size_t)(t0 + tt) * m.DP + idx] = v[tt];
    }
}

// ---------------------------------------------------------------------------------------------
// stage 3: recursion.  Workgroup 2b walks alpha of sequence b forward, workgroup 2b+1 walks beta
// backward.  Rows stored for frame t: alpha_t (state vector before frame t is consumed) and
// beta_{t+1} (after it), each relative to an offset kept in double precision.
// ---------------------------------------------------------------------------------------------
struct RecArgs {
    int T, B;
    const SeqMeta* meta; const uint2* ellA; const uint2* ellB; const float* gtab;
    float* alpha; float* beta; double* offA; double* offB;
};

// Barrier for LDS traffic only: waits for this wave's LDS operations and not for its global
// stores.  (On gfx9-family hardware loads and stores retire out of order with each other, so
// a wave that has both in flight can only wait for "all of them"; the recursion therefore
// keeps them in different waves: compute waves only store, the loader wave only loads.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Compute waves: thread tid owns states tid + j*THREADS.  Per frame: read the predecessor
// values and the staged emission scores from LDS, log-sum-exp in a fixed order, write the new
// value to the other LDS buffer and to the workspace row, one barrier.
template <int THREADS, int J, int KT>
__device__ __forceinline__ void recurse_compute(const RecArgs& a, const SeqMeta& m, const int b, const int dir,
                                                float* __restrict__ st0, float* __restrict__ st1,
                                                const float* __restrict__ am0, const float* __restrict__ am1,
                                                float* __restrict__ wmin) {
    constexpr int SCAP = THREADS * J, NW = THREADS / 64;
    const int tid = threadIdx.x;
    const int L = m.L, SP = m.SP, T = a.T;
    const long long soff = state_off(m.edge_begin, b);
    const uint2* ell = (dir ? a.ellB : a.ellA) + (size_t)KMAX * soff;
    float* ws = (dir ? a.beta : a.alpha) + (size_t)T * soff;
    double* offs = (dir ? a.offB : a.offA) + (size_t)b * T;
    const int K = dir ? m.Kout : m.Kin;

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
            eo[j][k] = other;
            es[j][k] = r.x >> 16;
            ew[j][k] = __uint_as_float(r.y);
        }
    }

    const int init_state = dir ? m.end_local : m.start_local;
    const int init_row = dir ? L - 1 : 0;
#pragma unroll
    for (int j = 0; j < J; j++) {
        const int s = tid + j * THREADS;
        const float v = s == init_state ? 0.f : INF_F;
        st0[s] = v;
        st1[s] = INF_F;
        if (s < SP) ws[(size_t)init_row * SP + s] = v;
    }
    if (tid < 16) { st0[SCAP + tid] = INF_F; st1[SCAP + tid] = INF_F; }
    if (tid == 0) offs[init_row] = 0.0;

    // step i consumes frame f(i) = i (alpha) or L-1-i (beta) and produces the row stored for
    // frame f(i)+1 (alpha) or f(i)-1 (beta)
    const int nsteps = L - 1;
    const long long wstep = dir ? -(long long)SP : (long long)SP;
    float* wp = ws + (size_t)init_row * SP + wstep;
    const int ostep = dir ? -1 : 1;
    double* op = offs + init_row + ostep;
    lds_barrier();

    double c = 0.0;
    bool pending = false;
    float* stc = st0; float* stn = st1;
    const float* amc = am0; const float* amn = am1;
    for (int i = 0; i < nsteps; i++) {
        float pend = 0.f;
        if (pending) {
            float mn = wmin[0];
#pragma unroll
            for (int w = 1; w < NW; w++) mn = fminf(mn, wmin[w]);
            pend = mn == INF_F ? 0.f : mn;
        }
        c += (double)pend;
        float rmin = INF_F;
#pragma unroll
        for (int j = 0; j < J; j++) {
            const int s = tid + j * THREADS;
            float v[KT];
            float mn = INF_F;
#pragma unroll
            for (int k = 0; k < KT; k++) {
                v[k] = (stc[eo[j][k]] - pend) + (ew[j][k] + amc[es[j][k]]);
                mn = fminf(mn, v[k]);
            }
            float sum = 0.f;
#pragma unroll
            for (int k = 0; k < KT; k++) sum += __builtin_amdgcn_exp2f((mn - v[k]) * 1.44269504088896341f);
            // sum is in [1, KT] whenever mn is finite: the raw log2 needs no range handling
            const float r = mn == INF_F ? INF_F : mn - 0.693147180559945309f * __builtin_amdgcn_logf(sum);
            stn[s] = r;
            if (s < SP) wp[s] = r;
            rmin = fminf(rmin, r);
        }
        if (tid == 0) *op = c;
        wp += wstep; op += ostep;
        pending = (i % RENORM) == RENORM - 1;
        if (pending) {
            rmin = wave_min(rmin);
            if ((tid & 63) == 0) wmin[tid >> 6] = rmin;
        }
        lds_barrier();
        float* t_ = stc; stc = stn; stn = t_;
        const float* u_ = amc; amc = amn; amn = u_;
    }
}

// Loader wave: keeps the compact emission rows of the next P frames in flight (registers)
// and drops the row of frame f(i+1) into the idle LDS buffer during step i.  It issues no
// global stores, so its loads retire in order and the wait counts stay exact.
template <int THREADS, int JL, int P>
__device__ __forceinline__ void recurse_load(const RecArgs& a, const SeqMeta& m, const int b, const int dir,
                                             float* __restrict__ am0, float* __restrict__ am1) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x - THREADS;
    const int L = m.L, DP = m.DP, T = a.T;
    const long long goff = slot_off(m.edge_begin, b);
    const float* G = a.gtab + (size_t)T * goff;
    const int nsteps = L - 1;
    const int nchunk = DP >> 2;                       // DP is a multiple of 16
    int cc[JL];                                       // my float4 chunks of a row (clamped)
#pragma unroll
    for (int jl = 0; jl < JL; jl++) cc[jl] = min(lane + jl * 64, nchunk - 1);
    // row consumed by step i (clamped to the steps that exist)
    auto rowp = [&](int i) -> const f4* {
        const int ic = min(i, nsteps - 1);
        return (const f4*)(G + (size_t)(dir ? L - 1 - ic : ic) * DP);
    };
    f4 g[P][JL];
    if (nsteps > 0) {
#pragma unroll
        for (int jl = 0; jl < JL; jl++) ((f4*)am0)[lane + jl * 64] = rowp(0)[cc[jl]];
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int jl = 0; jl < JL; jl++) g[p][jl] = rowp(1 + p)[cc[jl]];
    }
    lds_barrier();
    f4* amn = (f4*)am1; f4* amc = (f4*)am0;
    int i0 = 0;
    for (; i0 + P <= nsteps; i0 += P) {
#pragma unroll
        for (int q = 0; q < P; q++) {
            const f4* nxt = rowp(i0 + q + 1 + P);
#pragma unroll
            for (int jl = 0; jl < JL; jl++) {
                amn[lane + jl * 64] = g[q][jl];
                g[q][jl] = nxt[cc[jl]];
            }
            lds_barrier();
            f4* t_ = amc; amc = amn; amn = t_;
        }
    }
#pragma unroll
    for (int q = 0; q < P; q++) {
        if (i0 + q < nsteps) {
#pragma unroll
            for (int jl = 0; jl < JL; jl++) amn[lane + jl * 64] = g[q][jl];
            lds_barrier();
            f4* t_ = amc; amc = amn; amn = t_;
        }
    }
}

// THREADS compute threads plus one loader wave per workgroup.
template <int THREADS, int J, int JL, int P, int CLS>
__global__ __launch_bounds__(THREADS + 64) void fbw_recurse(RecArgs a) {
    constexpr int SCAP = THREADS * J, DCAP = 256 * JL, NW = THREADS / 64;
    __shared__ float st[2][SCAP + 16];
    __shared__ __attribute__((aligned(16))) float amr[2][DCAP];
    __shared__ float wmin[NW];

    const int b = blockIdx.x >> 1, dir = blockIdx.x & 1;
    const SeqMeta m = a.meta[b];
    if (rec_class(m) != CLS) return;
    if (threadIdx.x >= THREADS) {
        recurse_load<THREADS, JL, P>(a, m, b, dir, amr[0], amr[1]);
        return;
    }
    const int K = dir ? m.Kout : m.Kin;
    // the loop body is specialised on the number of edge slots per state so that all LDS
    // reads of a frame are issued back to back; unused slots point at the +inf cell
    if (K <= 2) recurse_compute<THREADS, J, 2>(a, m, b, dir, st[0], st[1], amr[0], amr[1], wmin);
    else if (K <= 3) recurse_compute<THREADS, J, 3>(a, m, b, dir, st[0], st[1], amr[0], amr[1], wmin);
    else if (K <= 4) recurse_compute<THREADS, J, 4>(a, m, b, dir, st[0], st[1], amr[0], amr[1], wmin);
    else if (K <= 6) recurse_compute<THREADS, J, 6>(a, m, b, dir, st[0], st[1], amr[0], amr[1], wmin);
    else recurse_compute<THREADS, J, KMAX>(a, m, b, dir, st[0], st[1], amr[0], amr[1], wmin);
}

// ---------------------------------------------------------------------------------------------
// stage 4: combine.  One workgroup per (strip of TC frames, sequence).  The F-wide row image
// lives in LDS: its non-hole positions are the same for every frame of a sequence, so it is
// filled once and only those positions are rewritten per frame before the row is streamed out.
// ---------------------------------------------------------------------------------------------
struct CombArgs {
    int T, B, F, out_mode;
    const SeqMeta* meta; const uint4* crec; const int* cbegin; const int* demis;
    const float* alpha; const float* beta; const float* gtab; const double* offA; const double* offB;
    float* out; float* sum_output;
    int xs_cap;
};

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float float4a __attribute__((ext_vector_type(4)));

__device__ inline void stream_const_row(float* dst, int F, float v) {
    const float4u c = {v, v, v, v};
    const int n4 = F >> 2;
    for (int i = threadIdx.x; i < n4; i += COMB_THREADS) __builtin_nontemporal_store(c, (float4u*)(dst + 4 * i));
    const int tail = F & 3;
    if ((int)threadIdx.x < tail) dst[4 * n4 + threadIdx.x] = v;
}

template <int CLS>
__global__ __launch_bounds__(COMB_THREADS) void fbw_combine(CombArgs a) {
    extern __shared__ float4a lds4[];
    __shared__ float redmin[COMB_THREADS / 64];
    __shared__ float redsum[COMB_THREADS / 64];
    constexpr int NW = COMB_THREADS / 64;

    const int b = blockIdx.y, t0 = blockIdx.x * TC, tid = threadIdx.x;
    const SeqMeta m = a.meta[b];
    if (comb_class(m) != CLS) return;
    const int T = a.T, B = a.B, F = a.F;
    const int t1 = min(T, t0 + TC);
    const bool prob = a.out_mode == I6FBW_OUT_PROB;
    const float hole = prob ? 0.f : INF_F;
    const int err = seq_error(m);
    const int L = (err || m.n_edges == 0) ? 0 : m.L;

    if (t0 >= L) {   // nothing but padding (or an unusable sequence) in this strip
        const float v = err ? __builtin_nanf("") : hole;
        for (int t = t0; t < t1; t++) {
            stream_const_row(a.out + ((size_t)t * B + b) * F, F, v);
            if (tid == 0) a.sum_output[(size_t)t * B + b] = err ? __builtin_nanf("") : 0.f;
        }
        return;
    }

    float* image = (float*)lds4;
    const int F4 = (F + 3) >> 2;
    float* xs = image + 4 * F4;
    for (int i = tid; i < F4; i += COMB_THREADS) lds4[i] = (float4a){hole, hole, hole, hole};

    const int nE = m.n_edges, D = m.D, SP = m.SP, DP = m.DP;
    const long long soff = state_off(m.edge_begin, b), goff = slot_off(m.edge_begin, b);
    const uint4* crec = a.crec + m.edge_begin;
    const int* cb = a.cbegin + goff;
    const int* de = a.demis + goff;
    const double* offA = a.offA + (size_t)b * T;
    const double* offB = a.offB + (size_t)b * T;

    for (int t = t0; t < t1; t++) {
        float* orow = a.out + ((size_t)t * B + b) * F;
        if (t >= L) {
            stream_const_row(orow, F, hole);
            if (tid == 0) a.sum_output[(size_t)t * B + b] = 0.f;
            continue;
        }
        const float* arow = a.alpha + (size_t)T * soff + (size_t)t * SP;
        const float* brow = a.beta + (size_t)T * soff + (size_t)t * SP;
        const float* grow = a.gtab + (size_t)T * goff + (size_t)t * DP;

        // edge scores x = alpha_t[from] + w + am + beta_{t+1}[to]   (fbw_op.cu:93-100)
        float lmin = INF_F;
        for (int i = tid; i < nE; i += COMB_THREADS) {
            const uint4 r = crec[i];
            const float x = arow[r.x & 0xFFFFu] + __uint_as_float(r.y) + grow[r.z] + brow[r.x >> 16];
            xs[i] = x;
            lmin = fminf(lmin, x);
        }
        lmin = wave_min(lmin);
        if ((tid & 63) == 0) redmin[tid >> 6] = lmin;
        __syncthreads();
        float mn = redmin[0];
#pragma unroll
        for (int w = 1; w < NW; w++) mn = fminf(mn, redmin[w]);
        const bool dead = mn == INF_F;
        for (int i = tid; i < nE; i += COMB_THREADS) xs[i] = dead ? 0.f : __expf(mn - xs[i]);
        __syncthreads();

        // per-emission sums in fixed (input) order, then the frame normaliser  (fbw_op.cu:115-134)
        float sd[COMB_JD];
        float lsum = 0.f;
#pragma unroll
        for (int jd = 0; jd < COMB_JD; jd++) {
            const int d = tid + jd * COMB_THREADS;
            float s = 0.f;
            if (d < D) {
                const int e0 = cb[d], e1 = cb[d + 1];
                for (int i = e0; i < e1; i++) s += xs[i];
            }
            sd[jd] = s;
            lsum += s;
        }
        lsum = wave_sum(lsum);
        if ((tid & 63) == 0) redsum[tid >> 6] = lsum;
        __syncthreads();
        float tot = redsum[0];
#pragma unroll
        for (int w = 1; w < NW; w++) tot += redsum[w];
        const float logtot = __logf(tot);
        if (tid == 0)
            a.sum_output[(size_t)t * B + b] = dead ? 0.f : (float)((double)(mn + -logtot) + offA[t] + offB[t]);
        const float inv = dead ? 0.f : 1.f / tot;
#pragma unroll
        for (int jd = 0; jd < COMB_JD; jd++) {
            const int d = tid + jd * COMB_THREADS;
            if (d < D) {
                float v;
                if (prob) v = sd[jd] * inv;
                else v = (dead || sd[jd] == 0.f) ? INF_F : logtot - __logf(sd[jd]);
                image[de[d]] = v;
            }
        }
        __syncthreads();
        const int n4 = F >> 2;
        for (int i = tid; i < n4; i += COMB_THREADS) __builtin_nontemporal_store((float4u)lds4[i], (float4u*)(orow + 4 * i));
        const int tail = F & 3;
        if (tid < tail) orow[4 * n4 + tid] = image[4 * n4 + tid];
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
thread_local hipError_t g_last_hip_error = hipSuccess;

struct Profile {
    bool on = false;
    int calls = 0;
    static constexpr int MAXREC = 256;
    hipEvent_t ev[MAXREC][I6FBW_N_STAGES + 1];
    bool created = false;
};
Profile g_prof;

#define HIP_TRY(expr)                                              \
    do {                                                           \
        hipError_t e_ = (expr);                                    \
        if (e_ != hipSuccess) { g_last_hip_error = e_; return I6FBW_ERR_LAUNCH; } \
    } while (0)

size_t comb_lds_bytes(int F, int xs_cap) { return (size_t)(((F + 3) >> 2) * 16) + (size_t)xs_cap * 4; }

}  // namespace

extern "C" {

int i6fbw_workspace_size(int T, int B, int F, int E, int n_states, size_t* bytes) {
    if (!bytes || T <= 0 || B <= 0 || F <= 0 || E < 0 || n_states <= 0) return I6FBW_ERR_INVALID_ARGUMENT;
    *bytes = make_layout(T, B, E).total;
    return I6FBW_OK;
}

int i6fbw_run(const float* am, int64_t am_stride_t, int64_t am_stride_b, const int32_t* edges, int64_t edge_row_stride,
              const float* weights, const int32_t* start_end, int64_t se_row_stride, const int32_t* seq_lens, int T,
              int B, int F, int E, int n_states, int out_mode, float* out, float* sum_output, void* workspace,
              size_t workspace_bytes, void* stream_) {
    if (T <= 0 || B <= 0 || F <= 0 || E < 0 || n_states <= 0) return I6FBW_ERR_INVALID_ARGUMENT;
    if (!am || !start_end || !seq_lens || !out || !sum_output || !workspace) return I6FBW_ERR_INVALID_ARGUMENT;
    if (E > 0 && (!edges || !weights)) return I6FBW_ERR_INVALID_ARGUMENT;
    if (out_mode != I6FBW_OUT_NEG_LOG && out_mode != I6FBW_OUT_PROB) return I6FBW_ERR_INVALID_ARGUMENT;
    if (((uintptr_t)workspace & 255) != 0) return I6FBW_ERR_INVALID_ARGUMENT;
    if (B > 65535) return I6FBW_ERR_INVALID_ARGUMENT;
    const Layout l = make_layout(T, B, E);
    if (workspace_bytes < l.total) return I6FBW_ERR_WORKSPACE_TOO_SMALL;
    const int xs_small = 1024, xs_large = EB_MAX;
    const bool need_large = E > 1024;
    if (F > F_BITMAP_MAX || comb_lds_bytes(F, need_large ? xs_large : xs_small) > 160 * 1024 - 256) return I6FBW_ERR_F_TOO_LARGE;

    hipStream_t stream = (hipStream_t)stream_;
    char* ws = (char*)workspace;
    SeqMeta* meta = (SeqMeta*)(ws + l.meta);

    hipEvent_t* ev = nullptr;
    if (g_prof.on) {
        if (!g_prof.created) {
            for (int i = 0; i < Profile::MAXREC; i++)
                for (int s = 0; s <= I6FBW_N_STAGES; s++) HIP_TRY(hipEventCreate(&g_prof.ev[i][s]));
            g_prof.created = true;
        }
        if (g_prof.calls < Profile::MAXREC) ev = g_prof.ev[g_prof.calls++];
    }
    if (ev) HIP_TRY(hipEventRecord(ev[0], stream));

    PrepArgs pa;
    pa.edges = edges; pa.edge_stride = edge_row_stride; pa.weights = weights;
    pa.start_end = start_end; pa.se_stride = se_row_stride; pa.seq_lens = seq_lens;
    pa.T = T; pa.B = B; pa.F = F; pa.E = E; pa.n_states = n_states;
    pa.meta = meta; pa.ellA = (uint2*)(ws + l.ellA); pa.ellB = (uint2*)(ws + l.ellB);
    pa.crec = (uint4*)(ws + l.crec); pa.cbegin = (int*)(ws + l.cbegin); pa.demis = (int*)(ws + l.demis);
    hipLaunchKernelGGL(fbw_prepare, dim3(3, B), dim3(1024), 0, stream, pa);
    HIP_TRY(hipGetLastError());
    if (ev) HIP_TRY(hipEventRecord(ev[1], stream));

    GatherArgs ga;
    ga.am = am; ga.st_t = am_stride_t; ga.st_b = am_stride_b; ga.T = T; ga.B = B;
    ga.meta = meta; ga.demis = pa.demis; ga.gtab = (float*)(ws + l.gtab);
    hipLaunchKernelGGL(fbw_gather, dim3((T + TG - 1) / TG, B), dim3(256), 0, stream, ga);
    HIP_TRY(hipGetLastError());
    if (ev) HIP_TRY(hipEventRecord(ev[2], stream));

    RecArgs ra;
    ra.T = T; ra.B = B; ra.meta = meta; ra.ellA = pa.ellA; ra.ellB = pa.ellB; ra.gtab = ga.gtab;
    ra.alpha = (float*)(ws + l.alpha); ra.beta = (float*)(ws + l.beta);
    ra.offA = (double*)(ws + l.offA); ra.offB = (double*)(ws + l.offB);
    hipLaunchKernelGGL((fbw_recurse<512, 1, 2, 8, 1>), dim3(2 * B), dim3(512 + 64), 0, stream, ra);
    HIP_TRY(hipGetLastError());
    // a sequence can only be in a larger class if the batch has that many states or emissions
    if (n_states > 512 || (E > 512 && F > 512)) {
        hipLaunchKernelGGL((fbw_recurse<512, 4, 8, 4, 2>), dim3(2 * B), dim3(512 + 64), 0, stream, ra);
        HIP_TRY(hipGetLastError());
    }
    if (n_states > 2048 || (E > 2048 && F > 2048)) {
        hipLaunchKernelGGL((fbw_recurse<512, 8, 16, 2, 3>), dim3(2 * B), dim3(512 + 64), 0, stream, ra);
        HIP_TRY(hipGetLastError());
    }
    if (ev) HIP_TRY(hipEventRecord(ev[3], stream));

    CombArgs ca;
    ca.T = T; ca.B = B; ca.F = F; ca.out_mode = out_mode;
    ca.meta = meta; ca.crec = pa.crec; ca.cbegin = pa.cbegin; ca.demis = pa.demis;
    ca.alpha = ra.alpha; ca.beta = ra.beta; ca.gtab = ga.gtab; ca.offA = ra.offA; ca.offB = ra.offB;
    ca.out = out; ca.sum_output = sum_output;
    static bool attr_set = false;
    if (!attr_set) {
        HIP_TRY(hipFuncSetAttribute((const void*)fbw_combine<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256));
        HIP_TRY(hipFuncSetAttribute((const void*)fbw_combine<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256));
        attr_set = true;
    }
    const dim3 cgrid((T + TC - 1) / TC, B);
    ca.xs_cap = xs_small;
    hipLaunchKernelGGL(fbw_combine<1>, cgrid, dim3(COMB_THREADS), comb_lds_bytes(F, xs_small), stream, ca);
    HIP_TRY(hipGetLastError());
    if (need_large) {
        ca.xs_cap = xs_large;
        hipLaunchKernelGGL(fbw_combine<2>, cgrid, dim3(COMB_THREADS), comb_lds_bytes(F, xs_large), stream, ca);
        HIP_TRY(hipGetLastError());
    }
    if (ev) HIP_TRY(hipEventRecord(ev[4], stream));
    return I6FBW_OK;
}

int i6fbw_read_status(const void* workspace, int B, void* stream, int* code, int* seq) {
    if (!workspace || B <= 0 || !code || !seq) return I6FBW_ERR_INVALID_ARGUMENT;
    SeqMeta* host = (SeqMeta*)malloc(sizeof(SeqMeta) * (size_t)B);
    if (!host) return I6FBW_ERR_INVALID_ARGUMENT;
    // the meta records sit at the start of the workspace
    hipError_t e = hipMemcpyAsync(host, workspace, sizeof(SeqMeta) * (size_t)B, hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) { g_last_hip_error = e; free(host); return I6FBW_ERR_LAUNCH; }
    *code = I6FBW_OK; *seq = -1;
    for (int b = 0; b < B; b++) {
        const int c = host[b].err ? host[b].err : (host[b].errA ? host[b].errA : host[b].errB);
        if (c) { *code = c; *seq = b; break; }
    }
    free(host);
    return I6FBW_OK;
}

const char* i6fbw_strerror(int code) {
    switch (code) {
        case I6FBW_OK: return "ok";
        case I6FBW_ERR_INVALID_ARGUMENT: return "invalid argument";
        case I6FBW_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
        case I6FBW_ERR_LAUNCH: return "HIP call failed";
        case I6FBW_ERR_F_TOO_LARGE: return "number of emission classes F exceeds the supported maximum";
        case I6FBW_ERR_SEQ_TOO_MANY_EDGES: return "a sequence has more edges than supported (8192)";
        case I6FBW_ERR_SEQ_SPARSE_STATES: return "state ids of a sequence span more than 2*edges+2 ids";
        case I6FBW_ERR_SEQ_DEGREE: return "a state has more than 8 incoming or outgoing edges";
        case I6FBW_ERR_SEQ_TOO_LARGE: return "a sequence has more than 4096 states or distinct emissions";
        case I6FBW_ERR_BAD_INDEX: return "sequence, emission or state index out of range";
        default: return "unknown status";
    }
}

const char* i6fbw_last_hip_error(void) { return g_last_hip_error == hipSuccess ? "" : hipGetErrorString(g_last_hip_error); }

void i6fbw_profile_enable(int on) {
    g_prof.on = on != 0;
    g_prof.calls = 0;
}

int i6fbw_profile_read(float* stage_ms) {
    const int n = g_prof.calls;
    for (int s = 0; s < I6FBW_N_STAGES; s++) stage_ms[s] = 0.f;
    if (n == 0) return 0;
    for (int i = 0; i < n; i++) {
        if (hipEventSynchronize(g_prof.ev[i][I6FBW_N_STAGES]) != hipSuccess) return 0;
        for (int s = 0; s < I6FBW_N_STAGES; s++) {
            float ms = 0.f;
            hipEventElapsedTime(&ms, g_prof.ev[i][s], g_prof.ev[i][s + 1]);
            stage_ms[s] += ms / n;
        }
    }
    g_prof.calls = 0;
    return n;
}

}  // extern "C"
