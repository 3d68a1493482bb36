/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the full-sum forward-backward (FBW) algorithm of
 * rwth-i6/i6_native_ops.  It exists only so that tests, the smoke check and the
 * benchmark's CPU-baseline leg have something to compare the HIP path with.
 * Nothing under i6_native_ops_amd/ may link, import or call it.
 *
 * The file is compiled twice: -DREAL=double gives the parity oracle
 * (fbw_oracle_f64), -DREAL=float gives the fp32 port used as the CPU baseline
 * (fbw_oracle_f32).  Both follow the reference's order of operations:
 *
 *   prob_add            i6_native_ops/fbw/fbw_op.cu:39-48
 *   alpha init          fbw_op.cu:296-302  (fill +inf, set_start_states :17-21)
 *   forward sweep       fbw_op.cu:318-333  (next_frame :71-102, fwd=true)
 *   beta seeding        fbw_op.cu:61-69,340-341 (init_bwd_state_buffer)
 *   backward sweep      fbw_op.cu:339-353  (next_frame with from/to swapped)
 *   per-frame normalise fbw_op.cu:104-135  (normalize)
 *   scatter to (T,B,F)  fbw_op.cu:137-153,366-377 (fill +inf, compute_result)
 *
 * The reference accumulates with an atomic CAS loop whose order is not
 * defined; this restatement accumulates in edge order.
 *
 * Pinning of this oracle (see tests/test_oracle_*.py): closed form on the
 * reference's own test fixture (test/fbw.py:9-41), brute-force path
 * enumeration on tiny automata, torch.nn.functional.ctc_loss on CTC
 * topologies, a dense log-semiring matrix chain via scipy logsumexp, finite
 * differences of the loss, and the row-sum invariant of test/fbw.py:60-64.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#ifndef REAL
#define REAL double
#endif
#ifndef SUFFIX
#define SUFFIX f64
#endif
#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

typedef REAL real;

/* float build uses the float libm entry points like the reference's device code */
static inline real r_exp(real x) { return sizeof(real) == 4 ? (real)expf((float)x) : (real)exp((double)x); }
static inline real r_log1p(real x) { return sizeof(real) == 4 ? (real)log1pf((float)x) : (real)log1p((double)x); }

/* fbw_op.cu:39-48 */
static inline real prob_add(real a, real b) {
    real diff = a - b;
    if (isnan(diff)) return (real)INFINITY;
    return -r_log1p(r_exp(-(real)fabs((double)diff))) + (a < b ? a : b);
}

typedef struct {
    const float* am; int64_t st_t, st_b;
    const int32_t *from, *to, *emis, *seq;
    const float* w;
    const int32_t *start, *end, *seq_lens;
    int T, B, F, n_states;
    float* out;            /* [T,B,F] contiguous, -log space, +inf holes */
    double* sum_output;    /* [T,B] */
} problem_t;

/*
 * Runs the whole algorithm for the edges idx[0..n) and the sequences
 * seqs[0..ns).  With all edges and all sequences this is exactly the
 * reference's global sweep; with the edges of one sequence it is that
 * sequence's share (automata of different sequences own disjoint states).
 */
static int run_subset(const problem_t* p, const int32_t* idx, int n, const int32_t* seqs, int ns) {
    const int T = p->T, B = p->B;
    uint32_t smin = 0xffffffffu, smax = 0;
    for (int i = 0; i < n; i++) {
        uint32_t f = (uint32_t)p->from[idx[i]], t = (uint32_t)p->to[idx[i]];
        if (f < smin) smin = f; if (f > smax) smax = f;
        if (t < smin) smin = t; if (t > smax) smax = t;
    }
    for (int i = 0; i < ns; i++) {
        uint32_t s = (uint32_t)p->start[seqs[i]], e = (uint32_t)p->end[seqs[i]];
        if (s < smin) smin = s; if (s > smax) smax = s;
        if (e < smin) smin = e; if (e > smax) smax = e;
    }
    if (smin > smax) return 0;
    if (smax >= (uint32_t)p->n_states) return -2;
    size_t ns_range = (size_t)smax - smin + 1;
    real* bufa = (real*)malloc(ns_range * sizeof(real));
    real* bufb = (real*)malloc(ns_range * sizeof(real));
    real* edge_buffer = (real*)malloc((size_t)T * (n > 0 ? n : 1) * sizeof(real));
    real* sum = (real*)malloc((size_t)B * sizeof(real));
    if (!bufa || !bufb || !edge_buffer || !sum) { free(bufa); free(bufb); free(edge_buffer); free(sum); return -1; }
    real *prev = bufa - smin, *next = bufb - smin;   /* index by global state id */
    const real INF = (real)INFINITY;

    /* fbw_op.cu:291-302 */
    for (size_t i = 0; i < (size_t)T * n; i++) edge_buffer[i] = 0;
    for (uint32_t s = smin; s <= smax; s++) prev[s] = INF;
    for (int i = 0; i < ns; i++) prev[(uint32_t)p->start[seqs[i]]] = 0;

    /* forward: fbw_op.cu:318-333 with next_frame(fwd=true) :71-102 */
    for (int t = 0; t < T; t++) {
        for (uint32_t s = smin; s <= smax; s++) next[s] = INF;
        real* eb = edge_buffer + (size_t)t * n;
        for (int i = 0; i < n; i++) {
            int e = idx[i];
            real pv = prev[(uint32_t)p->from[e]];
            if (isinf(pv)) { eb[i] = INF; continue; }
            real val = pv + (real)p->w[e] +
                       (real)p->am[t * p->st_t + (int64_t)(uint32_t)p->seq[e] * p->st_b + (uint32_t)p->emis[e]];
            eb[i] += val;
            uint32_t to = (uint32_t)p->to[e];
            next[to] = prob_add(next[to], val);
        }
        real* tmp = prev; prev = next; next = tmp;
    }

    /* backward: fbw_op.cu:336-353 */
    for (uint32_t s = smin; s <= smax; s++) prev[s] = INF;
    for (int t = T; t > 0; t--) {
        for (int i = 0; i < ns; i++) {            /* init_bwd_state_buffer :61-69 */
            int b = seqs[i];
            if ((uint32_t)(t - 1) + 1u == (uint32_t)p->seq_lens[b]) prev[(uint32_t)p->end[b]] = 0;
        }
        for (uint32_t s = smin; s <= smax; s++) next[s] = INF;
        real* eb = edge_buffer + (size_t)(t - 1) * n;
        for (int i = 0; i < n; i++) {
            int e = idx[i];
            real pv = prev[(uint32_t)p->to[e]];    /* from/to swapped :348 */
            if (isinf(pv)) { eb[i] = INF; continue; }
            real val = pv + (real)p->w[e] +
                       (real)p->am[(t - 1) * p->st_t + (int64_t)(uint32_t)p->seq[e] * p->st_b + (uint32_t)p->emis[e]];
            eb[i] += pv;
            uint32_t fr = (uint32_t)p->from[e];
            next[fr] = prob_add(next[fr], val);
        }
        real* tmp = prev; prev = next; next = tmp;
    }

    /* normalize :104-135 and compute_result :137-153 */
    for (int t = 0; t < T; t++) {
        real* eb = edge_buffer + (size_t)t * n;
        for (int i = 0; i < ns; i++) sum[seqs[i]] = INF;
        for (int i = 0; i < n; i++) {
            int b = (int)(uint32_t)p->seq[idx[i]];
            sum[b] = prob_add(sum[b], eb[i]);
        }
        for (int i = 0; i < ns; i++) {
            int b = seqs[i];
            p->sum_output[(size_t)t * B + b] = isinf(sum[b]) ? 0.0 : (double)sum[b];
        }
        for (int i = 0; i < n; i++) {
            int e = idx[i];
            uint32_t b = (uint32_t)p->seq[e];
            real score = eb[i] - sum[b];
            float* o = p->out + ((size_t)t * B + b) * p->F + (uint32_t)p->emis[e];
            *o = (float)prob_add((real)*o, score);
        }
    }
    free(bufa); free(bufb); free(edge_buffer); free(sum);
    return 0;
}

/*
 * am_scores [T,B,F] with strides st_t / st_b (elements); edges [4,E] with row
 * stride edge_stride (rows from,to,emission,seq: fbw_op.cu:249-256);
 * start_end [2,B] with row stride se_stride (:260-263).
 * out   float  [T,B,F] contiguous, -log posterior with +inf holes
 * loss  double [T,B]
 * threads <= 1: one global sweep over all edges in input order (the reference's
 *               exact structure).
 * threads  > 1: edges partitioned by sequence index, sequences processed
 *               concurrently (valid when automata own disjoint states).
 * Returns 0, -1 on allocation failure, -2 on an out-of-range index.
 */
int FN(fbw_oracle)(const float* am, int64_t st_t, int64_t st_b, const int32_t* edges, int64_t edge_stride,
                   const float* weights, const int32_t* start_end, int64_t se_stride, const int32_t* seq_lens,
                   int T, int B, int F, int E, int n_states, float* out, double* loss, int threads) {
    problem_t p;
    p.am = am; p.st_t = st_t; p.st_b = st_b;
    p.from = edges; p.to = edges + edge_stride; p.emis = edges + 2 * edge_stride; p.seq = edges + 3 * edge_stride;
    p.w = weights; p.start = start_end; p.end = start_end + se_stride; p.seq_lens = seq_lens;
    p.T = T; p.B = B; p.F = F; p.n_states = n_states; p.out = out; p.sum_output = loss;

    for (int e = 0; e < E; e++) {
        if ((uint32_t)p.seq[e] >= (uint32_t)B || (uint32_t)p.emis[e] >= (uint32_t)F) return -2;
    }
    /* fbw_op.cu:366-369: out <- +inf everywhere; sum_output starts at 0 (:232) */
    size_t n_out = (size_t)T * B * F;
    const float finf = INFINITY;
#pragma omp parallel for if (threads > 1) num_threads(threads > 1 ? threads : 1)
    for (size_t i = 0; i < n_out; i++) out[i] = finf;
    for (size_t i = 0; i < (size_t)T * B; i++) loss[i] = 0.0;

    int32_t* idx = (int32_t*)malloc(sizeof(int32_t) * (E > 0 ? E : 1));
    int32_t* seqs = (int32_t*)malloc(sizeof(int32_t) * (B > 0 ? B : 1));
    if (!idx || !seqs) { free(idx); free(seqs); return -1; }
    int rc = 0;
    if (threads <= 1) {
        for (int e = 0; e < E; e++) idx[e] = e;
        for (int b = 0; b < B; b++) seqs[b] = b;
        rc = run_subset(&p, idx, E, seqs, B);
    } else {
        int32_t* off = (int32_t*)calloc((size_t)B + 1, sizeof(int32_t));
        int32_t* cur = (int32_t*)malloc(sizeof(int32_t) * (size_t)(B + 1));
        if (!off || !cur) { free(off); free(cur); free(idx); free(seqs); return -1; }
        for (int e = 0; e < E; e++) off[(uint32_t)p.seq[e] + 1]++;
        for (int b = 0; b < B; b++) off[b + 1] += off[b];
        memcpy(cur, off, sizeof(int32_t) * (size_t)(B + 1));
        for (int e = 0; e < E; e++) idx[cur[(uint32_t)p.seq[e]]++] = e;   /* stable */
        for (int b = 0; b < B; b++) seqs[b] = b;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
        for (int b = 0; b < B; b++) {
            int r = run_subset(&p, idx + off[b], off[b + 1] - off[b], seqs + b, 1);
            if (r != 0) {
#pragma omp critical
                rc = r;
            }
        }
        free(off); free(cur);
    }
    free(idx); free(seqs);
    return rc;
}

#ifdef ORACLE_COMMON
int fbw_oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
#endif
