/*
 * cf_oracle_moe_bwd.c -- CPU restatement of the custom kernels of the MoE
 * expert-bank backward with forward-owned routes (src/trainer.cu:7654-7741):
 * exact-erf GELU forward and backward, the per-row dot with the expert's
 * output, the route-weighted gather of the upstream gradient and the
 * scatter-add of the expert's input gradient.
 *
 * TEST INFRASTRUCTURE ONLY (see cf_oracle.h).
 *
 * Pinning status:
 *   orc_moe_row_dot_selected_bf16   products of two bf16 values are exact in
 *                          fp32, so only the summation tree matters: per-thread
 *                          strided partial sums, then the shared-memory halving
 *                          tree (stride T/2 .. 1).  Pinned by rows whose sums are
 *                          exact in any order (small integers), by a double
 *                          recomputation, by a crafted row on which a sequential
 *                          sum differs, and by H = 192, where the halving tree of
 *                          a launch of 192 threads leaves out the partials of
 *                          threads 2, 5, 8, ... as the reference source does.
 *                          The reference holds no test vector for this kernel.
 *   orc_moe_gather_scale_rows_bf16, orc_moe_scatter_add_rows_bf16
 *                          one IEEE operation and one bf16 rounding per element:
 *                          closed forms and permutation identities.
 *   orc_gelu_forward_bf16, orc_gelu_backward_bf16
 *                          libm erff / expf stand in for CUDA's: double
 *                          recomputation to half a bf16 ulp, the derivative
 *                          against a central difference of the forward in
 *                          double, gelu'(0) = 1/2, odd/even symmetries.
 *                          Parity unpinned beyond one bf16 ulp.
 */
#include "cf_oracle.h"

#include <math.h>
#include <stdlib.h>

/* kernels/moe.cu:510-521 */
void orc_gelu_forward_bf16(const uint16_t* x, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        const float v = orc_bf16_to_f32(x[i]);
        const float g = 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
        out[i] = orc_bf16_from_f32(g);
    }
}

/* kernels/moe.cu:1148-1167; `cdf + x * pdf` is one fused multiply-add under nvcc's default contraction */
void orc_gelu_backward_bf16(const uint16_t* pre, const uint16_t* d_post, uint16_t* d_pre, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        const float x = orc_bf16_to_f32(pre[i]);
        const float cdf = 0.5f * (1.0f + erff(x * 0.7071067811865476f));
        const float pdf = 0.3989422804014327f * expf(-0.5f * x * x);
        const float deriv = fmaf(x, pdf, cdf);
        d_pre[i] = orc_bf16_from_f32(orc_bf16_to_f32(d_post[i]) * deriv);
    }
}

/* kernels/moe.cu:623-645 (kernel), :740-748 (launch: T = min(H, 256) threads, one block per compact row) */
void orc_moe_row_dot_selected_bf16(const uint16_t* a_full, const uint16_t* b_compact, float* out,
                                   const int* row_indices, int n_rows, int H, int out_stride, int out_col) {
    const int T = H < 256 ? H : 256;
    if (T <= 0) return;
    float sh[256];
    for (int i = 0; i < n_rows; ++i) {
        const int row = row_indices[i];
        const uint16_t* a = a_full + (size_t)row * H;
        const uint16_t* b = b_compact + (size_t)i * H;
        for (int t = 0; t < T; ++t) {
            float sum = 0.0f;
            for (int h = t; h < H; h += T) sum = fmaf(orc_bf16_to_f32(a[h]), orc_bf16_to_f32(b[h]), sum);
            sh[t] = sum;
        }
        for (int stride = T / 2; stride > 0; stride >>= 1)
            for (int t = 0; t < stride; ++t) sh[t] += sh[t + stride];
        out[(size_t)row * out_stride + out_col] = sh[0];
    }
}

/* kernels/moe.cu:646-660, :750-758 */
void orc_moe_gather_scale_rows_bf16(const uint16_t* src, uint16_t* dst, const float* route_weights,
                                    const int* row_indices, int n_rows, int expert_idx, int num_experts, int H) {
    for (int i = 0; i < n_rows; ++i) {
        const int row = row_indices[i];
        const float w = route_weights[(size_t)row * num_experts + expert_idx];
        for (int h = 0; h < H; ++h)
            dst[(size_t)i * H + h] = orc_bf16_from_f32(w * orc_bf16_to_f32(src[(size_t)row * H + h]));
    }
}

/* kernels/moe.cu:661-674, :760-767 */
void orc_moe_scatter_add_rows_bf16(uint16_t* dst_full, const uint16_t* src_compact, const int* row_indices,
                                   int n_rows, int H) {
    for (int i = 0; i < n_rows; ++i) {
        uint16_t* d = dst_full + (size_t)row_indices[i] * H;
        for (int h = 0; h < H; ++h)
            d[h] = orc_bf16_from_f32(orc_bf16_to_f32(d[h]) + orc_bf16_to_f32(src_compact[(size_t)i * H + h]));
    }
}
