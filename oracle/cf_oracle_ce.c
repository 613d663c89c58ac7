/*
 * cf_oracle_ce.c -- CPU restatement of the chunked cross-entropy forward +
 * backward (kernels/cross_entropy.cu:9-44, 201-305).
 *
 * TEST INFRASTRUCTURE ONLY (see cf_oracle.h).
 *
 * The restatement keeps the reference's structure: 128 threads per row, each
 * summing exp(logit - max) over the columns t, t + 128, ..., a 32-lane xor
 * butterfly, then a butterfly over the four leaders.  exp and log are libm's
 * (correctly rounded to within an ulp); CUDA's expf / logf differ from them
 * in the last bits, so this oracle defines the gradient to within one bf16
 * ulp, not to the bit: the HIP kernel (hardware exp2 / log2) is compared
 * with that tolerance, and both against a double-precision softmax.
 * Pinning: closed forms (uniform logits, one dominant logit), sum-to-zero of
 * every gradient row, double-precision recomputation.  The reference holds
 * no test vector for this kernel: parity unpinned beyond that tolerance.
 */
#include "cf_oracle.h"

#include <float.h>
#include <math.h>

static float butterfly32_sum(float* v) {
    for (int off = 16; off > 0; off >>= 1) {
        float next[32];
        for (int i = 0; i < 32; ++i) next[i] = v[i] + v[i ^ off];
        for (int i = 0; i < 32; ++i) v[i] = next[i];
    }
    return v[0];
}

/* kernels/cross_entropy.cu:201-219, 281-287: accumulates into *n_valid (the caller zeroes it) */
void orc_cross_entropy_count_valid(const int32_t* labels, int n, int* n_valid) {
    for (int i = 0; i < n; ++i) if (labels[i] >= 0) ++*n_valid;
}

/* kernels/cross_entropy.cu:225-305 (k_ce_fwd_bwd_scaled, 128 threads per row).  grad may alias logits. */
void orc_cross_entropy_fwd_bwd_chunk(const uint16_t* logits, const int32_t* labels, float* loss_out,
                                     uint16_t* grad, int rows, int V, const int* n_valid) {
    enum { T = 128 };
    const int nv = *n_valid > 1 ? *n_valid : 1;
    const float inv_n = 1.0f / (float)nv;                                       /* :244 */
    for (int row = 0; row < rows; ++row) {
        const uint16_t* lr = logits + (size_t)row * V;
        uint16_t* gr = grad + (size_t)row * V;
        const int label = labels[row];
        if (label < 0) {                                                        /* :237-241 */
            for (int v = 0; v < V; ++v) gr[v] = 0;
            continue;
        }
        float row_max = -FLT_MAX;                                               /* :247-255, order-free */
        for (int v = 0; v < V; ++v) {
            const float lv = orc_bf16_to_f32(lr[v]);
            if (lv > row_max) row_max = lv;
        }
        float part[T];                                                          /* :257-260 */
        for (int t = 0; t < T; ++t) {
            float s = 0.0f;
            for (int v = t; v < V; v += T) s += expf(orc_bf16_to_f32(lr[v]) - row_max);
            part[t] = s;
        }
        float leaders[32];                                                      /* :33-43 */
        for (int w = 0; w < 32; ++w) leaders[w] = 0.0f;
        for (int w = 0; w < T / 32; ++w) leaders[w] = butterfly32_sum(part + 32 * w);
        const float sum = butterfly32_sum(leaders);
        const float inv_sum = 1.0f / sum;                                       /* :266 */
        float label_log_prob = 0.0f;
        for (int v = 0; v < V; ++v) {                                           /* :270-276 */
            const float prob = expf(orc_bf16_to_f32(lr[v]) - row_max) * inv_sum;
            const float gv = (prob - (v == label ? 1.0f : 0.0f)) * inv_n;
            if (v == label) label_log_prob = logf(prob + 1e-9f);
            gr[v] = orc_bf16_from_f32(gv);
        }
        *loss_out += -label_log_prob * inv_n;                                   /* :279-280 (atomicAdd: row order is free) */
    }
}
