/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the best-path (Viterbi) alignment of rwth-i6/i6_native_ops, in the
 * reference's own arithmetic (fp32, the same order of additions), so that scores and
 * back-pointers can be compared bit for bit.  Nothing under i6_native_ops_amd/ may link,
 * import or call it.
 *
 *   buffer init (-inf, -1)     i6_native_ops/fast_viterbi/core.cu:51-63,209-211
 *   start states               core.cu:65-78
 *   one frame over all edges   core.cu:80-122  (only edges of sequences with t < seq_len;
 *                              candidate = prev + weight + am[t, seq, emission], maximised)
 *   tie rule                   core.cu:20-49   (larger value wins; equal values: the smaller
 *                              edge index wins; a candidate of -inf never replaces (-inf, -1))
 *   score                      core.cu:124-143 (value of the end state in frame seq_len)
 *   back-trace                 core.cu:145-177,246-264 (from the end state; a state without a
 *                              back-pointer emits 0 and stays where it is; frames >= seq_len emit 0)
 *
 * Outside the reference's defined behaviour: seq_len > T reads past its buffer there; here
 * seq_len is clamped to [0, T].
 *
 * Pinning (tests/test_oracle_viterbi.py): the reference's own test vector
 * (test/fast_viterbi.py:9-39), brute-force enumeration of all paths on tiny automata, hand-worked
 * tie cases.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

typedef struct { int32_t idx; float val; } IdxVal;

int viterbi_oracle_f32(const float* am, int64_t st_t, int64_t st_b, const int32_t* edges, int64_t edge_stride,
                       const float* weights, const int32_t* start_end, int64_t se_stride, const int32_t* seq_lens,
                       int T, int B, int F, int E, int n_states, int32_t* alignment /* [T,B] */, float* scores /* [B] */) {
    (void)F;
    const int32_t* e_from = edges;
    const int32_t* e_to = edges + edge_stride;
    const int32_t* e_emis = edges + 2 * edge_stride;
    const int32_t* e_seq = edges + 3 * edge_stride;
    IdxVal* buf = (IdxVal*)malloc(sizeof(IdxVal) * (size_t)(T + 1) * (size_t)n_states);
    int32_t* cur = (int32_t*)malloc(sizeof(int32_t) * (size_t)B);
    if (!buf || !cur) { free(buf); free(cur); return -1; }
    for (size_t i = 0; i < (size_t)(T + 1) * (size_t)n_states; i++) { buf[i].idx = -1; buf[i].val = -INFINITY; }
    for (int b = 0; b < B; b++) buf[start_end[b]].val = 0.f;

    for (int t = 0; t < T; t++) {
        const IdxVal* prev = buf + (size_t)t * n_states;
        IdxVal* next = buf + (size_t)(t + 1) * n_states;
        for (int e = 0; e < E; e++) {
            const int seq = e_seq[e];
            if (t >= seq_lens[seq]) continue;
            /* two additions, left to right, as in the reference */
            float cand = prev[e_from[e]].val + weights[e];
            cand = cand + am[(int64_t)t * st_t + (int64_t)seq * st_b + e_emis[e]];
            IdxVal* a = next + e_to[e];
            if (cand < a->val) continue;
            if (cand == a->val && e >= a->idx) continue;
            a->val = cand;
            a->idx = e;
        }
    }
    for (int b = 0; b < B; b++) {
        int len = seq_lens[b];
        if (len < 0) len = 0;
        if (len > T) len = T;
        scores[b] = buf[(size_t)len * n_states + start_end[se_stride + b]].val;
        cur[b] = start_end[se_stride + b];
    }
    for (int t = T - 1; t >= 0; t--) {
        const IdxVal* frame = buf + (size_t)(t + 1) * n_states;
        for (int b = 0; b < B; b++) {
            int32_t out = 0;
            if (t < seq_lens[b]) {
                const int e = frame[cur[b]].idx;
                if (e >= 0) { cur[b] = e_from[e]; out = e_emis[e]; }
            }
            alignment[(size_t)t * B + b] = out;
        }
    }
    free(buf); free(cur);
    return 0;
}
