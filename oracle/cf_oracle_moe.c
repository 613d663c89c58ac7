/*
 * cf_oracle_moe.c -- CPU restatement of the reference MoE routing / dispatch
 * path.  TEST INFRASTRUCTURE ONLY (see cf_oracle.h).  Build with
 * -ffp-contract=off.
 */
#include "cf_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- expf -----------------------------------------------------------------
 * The router and the SiLU gate call the device expf (kernels/cross_entropy.cu:
 * 179,187; kernels/activations.cu:13-15).  CUDA's expf is not bit-specified,
 * so this build fixes one: Cody-Waite reduction by ln2 in two pieces, a
 * degree-6 polynomial evaluated with explicit fused multiply-adds, exact
 * power-of-two scaling with gradual underflow.  Only IEEE-exact operations
 * are used, so the device kernel that repeats these steps returns the same
 * bits. */
float orc_expf(float x) {
    if (x != x) return x;
    if (x > 88.72284f) return INFINITY;
    if (x < -103.97208f) return 0.0f;
    const float k = rintf(x * 1.44269504f);
    float r = fmaf(k, -0.693359375f, x);
    r = fmaf(k, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    p = fmaf(p, r * r, r);
    p = p + 1.0f;
    const int ki = (int)k;
    if (ki < -126) return (p * u2f((uint32_t)(ki + 100 + 127) << 23)) * 7.8886090522101181e-31f; /* 2^-100 */
    if (ki > 127)  return (p * u2f((uint32_t)(ki - 1 + 127) << 23)) * 2.0f;
    return p * u2f((uint32_t)(ki + 127) << 23);
}
void orc_expf_n(const float* in, float* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_expf(in[i]); }

/* ---- softmax ---------------------------------------------------------------
 * kernels/cross_entropy.cu:167-197 with the reduction order of its launch:
 * T = min(cols,256) threads; thread t accumulates columns t, t+T, ... in
 * order; each 32-lane group is combined by an xor butterfly (offsets 16..1,
 * kernels/cross_entropy.cu:15-19); the per-group sums are combined by one more
 * butterfly with absent lanes contributing 0 (kernels/cross_entropy.cu:35-45).
 * Lanes that do not exist (T not a multiple of 32) contribute 0. */
static float butterfly32(float* v) {
    for (int off = 16; off > 0; off >>= 1) {
        float t[32];
        for (int l = 0; l < 32; ++l) t[l] = v[l] + v[l ^ off];
        memcpy(v, t, sizeof(t));
    }
    return v[0];
}
void orc_softmax_inplace_f32(float* x, int rows, int cols) {
    if (cols <= 0) return;
    const int T = cols < 256 ? cols : 256;
    const int nwarps = (T + 31) / 32;
    for (int row = 0; row < rows; ++row) {
        float* r = x + (size_t)row * cols;
        float mx = -3.402823466e+38f;
        for (int c = 0; c < cols; ++c) mx = fmaxf(mx, r[c]);
        float warp_sum[32];
        for (int w = 0; w < 32; ++w) warp_sum[w] = 0.0f;
        for (int w = 0; w < nwarps; ++w) {
            float lane[32];
            for (int l = 0; l < 32; ++l) {
                const int t = w * 32 + l;
                float s = 0.0f;
                if (t < T) for (int c = t; c < cols; c += T) s += orc_expf(r[c] - mx);
                lane[l] = s;
            }
            warp_sum[w] = butterfly32(lane);
        }
        const float sum = butterfly32(warp_sum);
        const float inv = 1.0f / sum;
        for (int c = 0; c < cols; ++c) r[c] = orc_expf(r[c] - mx) * inv;
    }
}

/* ---- top-k -----------------------------------------------------------------
 * kernels/moe.cu:374-422.  The reference keeps its flags in bool kept[32]
 * (kernels/moe.cu:383), which is too small for 64 experts; the flags here are
 * sized by num_experts, everything else is the same: strict > against -1 so
 * the lowest index wins ties, kept sum in ascending expert order. */
void orc_moe_topk_route_f32(float* scores, int rows, int num_experts, int top_k,
                            float* row_sum_save, float* scores_save, int normalize_topk) {
    orc_softmax_inplace_f32(scores, rows, num_experts);
    if (scores_save) memcpy(scores_save, scores, (size_t)rows * num_experts * sizeof(float));
    unsigned char* kept = (unsigned char*)malloc((size_t)(num_experts > 0 ? num_experts : 1));
    const int k = top_k < num_experts ? top_k : num_experts;
    for (int row = 0; row < rows; ++row) {
        float* s = scores + (size_t)row * num_experts;
        memset(kept, 0, (size_t)num_experts);
        for (int pick = 0; pick < k; ++pick) {
            int best = -1;
            float best_v = -1.0f;
            for (int e = 0; e < num_experts; ++e)
                if (!kept[e] && s[e] > best_v) { best_v = s[e]; best = e; }
            if (best < 0) break;
            kept[best] = 1;
        }
        float sum = 0.0f;
        for (int e = 0; e < num_experts; ++e) if (kept[e]) sum += s[e];
        if (row_sum_save) row_sum_save[row] = sum;
        const float inv_sum = (normalize_topk && sum > 0.0f) ? (1.0f / sum) : 1.0f;
        for (int e = 0; e < num_experts; ++e) s[e] = kept[e] ? s[e] * inv_sum : 0.0f;
    }
    free(kept);
}

/* ---- dispatch ---------------------------------------------------------------
 * kernels/moe.cu:565-580,702-710.  Membership is weight > 0; row_indices is
 * expert-major with stride `rows`.  The reference fills each list in atomicAdd
 * arrival order (kernels/moe.cu:576-577); the canonical order here is ascending
 * row, and equality with the reference is as a set per expert. */
void orc_moe_build_expert_row_lists(const float* route_weights, int* counts, int* row_indices,
                                    int rows, int num_experts) {
    for (int e = 0; e < num_experts; ++e) counts[e] = 0;
    for (int row = 0; row < rows; ++row) {
        const float* rw = route_weights + (size_t)row * num_experts;
        for (int e = 0; e < num_experts; ++e)
            if (rw[e] > 0.0f) row_indices[(size_t)e * rows + counts[e]++] = row;
    }
}

/* kernels/moe.cu:785-795 */
void orc_moe_expert_offsets_from_counts(const int* counts, int* offsets, int num_experts) {
    int sum = 0;
    for (int e = 0; e < num_experts; ++e) { offsets[e] = sum; sum += counts[e]; }
}

/* kernels/moe.cu:594-606 */
void orc_moe_gather_rows_u8(const uint8_t* src, uint8_t* dst, const int* row_indices,
                            int n_rows, int width) {
    for (int i = 0; i < n_rows; ++i)
        memcpy(dst + (size_t)i * width, src + (size_t)row_indices[i] * width, (size_t)width);
}
/* kernels/moe.cu:581-593 */
void orc_moe_gather_rows_bf16(const uint16_t* src, uint16_t* dst, const int* row_indices,
                              int n_rows, int width) {
    for (int i = 0; i < n_rows; ++i)
        memcpy(dst + (size_t)i * width, src + (size_t)row_indices[i] * width, (size_t)width * 2);
}

/* kernels/moe.cu:607-622: `mixed + w * compact` in fp32, then one bf16 rounding.  The reference builds
 * its device code with the CUDA compiler's defaults (no -fmad=false in CMakeLists.txt), which contract
 * a multiply feeding an add into one fused multiply-add, so the restatement is fmaf. */
void orc_moe_scatter_accumulate_rows_bf16(uint16_t* mixed, const uint16_t* compact,
                                          const float* route_weights, const int* row_indices,
                                          int n_rows, int expert_idx, int num_experts, int H) {
    for (int i = 0; i < n_rows; ++i) {
        const int row = row_indices[i];
        const float w = route_weights[(size_t)row * num_experts + expert_idx];
        for (int h = 0; h < H; ++h) {
            uint16_t* dst = mixed + (size_t)row * H + h;
            *dst = orc_bf16_from_f32(fmaf(w, orc_bf16_to_f32(compact[(size_t)i * H + h]), orc_bf16_to_f32(*dst)));
        }
    }
}

/* kernels/moe.cu:529-542 (same contraction as above) */
void orc_moe_scale_accumulate_bf16(uint16_t* mixed, const uint16_t* term,
                                   const float* route_weights, int rows, int expert_idx,
                                   int num_experts, int H) {
    for (int row = 0; row < rows; ++row) {
        const float w = route_weights[(size_t)row * num_experts + expert_idx];
        for (int h = 0; h < H; ++h) {
            uint16_t* dst = mixed + (size_t)row * H + h;
            *dst = orc_bf16_from_f32(fmaf(w, orc_bf16_to_f32(term[(size_t)row * H + h]), orc_bf16_to_f32(*dst)));
        }
    }
}

/* ---- grouped GELU expert bank -------------------------------------------------
 * kernels/moe.cu:950-1060: per selected (expert,row): dequantise hidden and
 * weights with their per-tensor descales, fc_in, exact-erf GELU kept in
 * floating point (not re-quantised, kernels/moe.cu:893-903), fc_out, multiply
 * by the route weight, add into mixed.  The reference adds with a bf16
 * compare-and-swap whose order is scheduling dependent; this reference
 * accumulates in double so a device result can be compared with a tolerance. */
typedef struct {
    const uint8_t* hidden; float dh; int e5m2;
    const float* rw; const int* counts; const int* idx;
    const uint8_t* w_in; float din; const uint8_t* w_out; float dout;
    double* mixed; int rows, H, Ie, E, e0, e1;
} grouped_job;

static void* grouped_worker(void* arg) {
    grouped_job* j = (grouped_job*)arg;
    float lut_h[256], lut_w[256];
    for (int b = 0; b < 256; ++b) {
        lut_h[b] = (j->e5m2 ? orc_e5m2_unpack((uint8_t)b) : orc_e4m3_unpack((uint8_t)b));
        lut_w[b] = orc_e4m3_unpack((uint8_t)b);
    }
    double* act = (double*)malloc(sizeof(double) * (size_t)j->Ie);
    float* hrow = (float*)malloc(sizeof(float) * (size_t)j->H);
    /* a worker owns a contiguous range of ROWS so no two workers touch one output row */
    for (int e = 0; e < j->E; ++e) {
        const uint8_t* win = j->w_in + (size_t)e * j->H * j->Ie;
        const uint8_t* wout = j->w_out + (size_t)e * j->Ie * j->H;
        for (int s = 0; s < j->counts[e]; ++s) {
            const int row = j->idx[(size_t)e * j->rows + s];
            if (row < j->e0 || row >= j->e1) continue;
            for (int k = 0; k < j->H; ++k) hrow[k] = lut_h[j->hidden[(size_t)row * j->H + k]] * j->dh;
            for (int i = 0; i < j->Ie; ++i) {
                double acc = 0.0;
                for (int k = 0; k < j->H; ++k)
                    acc += (double)hrow[k] * (double)(lut_w[win[(size_t)i * j->H + k]] * j->din);
                act[i] = 0.5 * acc * (1.0 + erf(acc * 0.70710678118654752440));
            }
            const double w = (double)j->rw[(size_t)row * j->E + e];
            for (int h = 0; h < j->H; ++h) {
                double acc = 0.0;
                for (int i = 0; i < j->Ie; ++i)
                    acc += act[i] * (double)(lut_w[wout[(size_t)h * j->Ie + i]] * j->dout);
                j->mixed[(size_t)row * j->H + h] += w * acc;
            }
        }
    }
    free(act); free(hrow);
    return NULL;
}

void orc_moe_grouped_expert_forward_fp8_ref(
    const uint8_t* hidden, float fcin_descale, int fcin_is_e5m2,
    const float* route_weights, const int* counts, const int* row_indices,
    const uint8_t* fc_in_w, float fc_in_descale,
    const uint8_t* fc_out_w, float fc_out_descale,
    double* mixed_ref, int rows, int H, int Ie, int num_experts, int threads) {
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    pthread_t tid[64];
    grouped_job jobs[64];
    for (int t = 0; t < threads; ++t) {
        grouped_job j = { hidden, fcin_descale, fcin_is_e5m2, route_weights, counts, row_indices,
                          fc_in_w, fc_in_descale, fc_out_w, fc_out_descale, mixed_ref,
                          rows, H, Ie, num_experts,
                          (int)((long long)rows * t / threads), (int)((long long)rows * (t + 1) / threads) };
        jobs[t] = j;
        pthread_create(&tid[t], NULL, grouped_worker, &jobs[t]);
    }
    for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
}
