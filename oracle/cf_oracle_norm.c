/*
 * cf_oracle_norm.c -- CPU restatement of the producers that feed the FP8
 * quantizer: RMSNorm forward and the absolute-ceiling activation row clip.
 *
 * TEST INFRASTRUCTURE ONLY (see cf_oracle.h).
 *
 * Both reference kernels reduce a row with a fixed tree: a per-thread strided
 * partial sum (nvcc contracts `s += v * v` into one fused multiply-add), a
 * 32-lane xor butterfly, then a second stage over the warp leaders.  The
 * restatement walks exactly that tree, so the bf16 outputs are defined bit for
 * bit by the reference source, not merely to rounding error.
 *
 * Pinning status:
 *   orc_rmsnorm_forward    closed forms (a constant row, a one-hot row, a row
 *                          of +-1 whose sum of squares is exact in any order),
 *                          double-precision recomputation within 1 bf16 ulp,
 *                          and a crafted row on which a sequential sum gives a
 *                          different bf16 output than the tree (the test is
 *                          sensitive to the order).  The reference holds no
 *                          test vector for this kernel: beyond the source text
 *                          the summation order is parity unpinned.
 *   orc_act_row_clip_abs   same scheme; rows at or under the ceiling are left
 *                          untouched bit for bit.
 */
#include "cf_oracle.h"

#include <math.h>
#include <stdlib.h>

/* lane 0 of a 32-lane xor butterfly (offsets 16, 8, 4, 2, 1); v is clobbered */
static float butterfly32(float* v) {
    for (int off = 16; off > 0; off >>= 1) {
        float next[32];
        for (int i = 0; i < 32; ++i) next[i] = v[i] + v[i ^ off];
        for (int i = 0; i < 32; ++i) v[i] = next[i];
    }
    return v[0];
}

/* kernels/rmsnorm.cu:13-54 (kernel), :101-108 (launch: T = min(H, 512) threads, one block per row).
 * T must be a multiple of 32 (the reference shuffles with a full mask). */
int orc_rmsnorm_forward(const uint16_t* x, const uint16_t* scale, uint16_t* out, float* rms,
                        int rows, int H, float eps) {
    const int T = H < 512 ? H : 512;
    if (T <= 0 || T % 32 != 0) return -1;
    const int nwarps = T / 32;
    float* part = (float*)malloc(sizeof(float) * (size_t)T);
    if (!part) return -2;
    for (int row = 0; row < rows; ++row) {
        const uint16_t* xr = x + (size_t)row * H;
        uint16_t* orow = out + (size_t)row * H;
        /* :24-28 per-thread strided partials */
        for (int t = 0; t < T; ++t) {
            float ms = 0.0f;
            for (int h = t; h < H; h += T) {
                const float v = orc_bf16_to_f32(xr[h]);
                ms = fmaf(v, v, ms);
            }
            part[t] = ms;
        }
        /* :30-31 warp butterflies, :34-41 the first warp reduces the leaders (absent warps count 0) */
        float leaders[32];
        for (int w = 0; w < 32; ++w) leaders[w] = 0.0f;
        for (int w = 0; w < nwarps; ++w) leaders[w] = butterfly32(part + 32 * w);
        const float total = butterfly32(leaders);
        /* :44-45 */
        const float rms_val = sqrtf(total / (float)H + eps);
        if (rms) rms[row] = rms_val;
        /* :48-52 */
        const float inv_rms = 1.0f / rms_val;
        for (int h = 0; h < H; ++h) {
            const float v = orc_bf16_to_f32(xr[h]) * inv_rms * orc_bf16_to_f32(scale[h]);
            orow[h] = orc_bf16_from_f32(v);
        }
    }
    free(part);
    return 0;
}

/* src/trainer.cu:3822-3842 (k_act_row_normsq, 256 threads), :3940-3958 (k_act_row_clip_apply_abs),
 * :3968-3991 (act_row_clip, fixed mode: ceiling <= 0 disables).  normsq[rows] receives the row sums of
 * squares as the reference's scratch does; may be NULL. */
void orc_act_row_clip_abs(uint16_t* x, int rows, int cols, float ceiling, float* normsq) {
    if (ceiling <= 0.0f) return;
    for (int row = 0; row < rows; ++row) {
        uint16_t* xr = x + (size_t)row * cols;
        float part[256];
        for (int t = 0; t < 256; ++t) {
            float s = 0.0f;
            for (int c = t; c < cols; c += 256) {
                const float v = orc_bf16_to_f32(xr[c]);
                s = fmaf(v, v, s);
            }
            part[t] = s;
        }
        float total = 0.0f;                       /* :3837-3839 thread 0 adds the eight leaders in order */
        for (int w = 0; w < 8; ++w) total += butterfly32(part + 32 * w);
        if (normsq) normsq[row] = total;
        const float norm = sqrtf(total);
        if (norm <= ceiling) continue;            /* :3953 (a NaN norm fails this test and poisons the row, as in the reference) */
        const float scalef = ceiling / norm;
        for (int c = 0; c < cols; ++c) xr[c] = orc_bf16_from_f32(orc_bf16_to_f32(xr[c]) * scalef);
    }
}
