/*
 * cf_oracle.c -- CPU restatement of the reference FP8 quantize path.
 * TEST INFRASTRUCTURE ONLY (see cf_oracle.h).  Build with -ffp-contract=off.
 */
#include "cf_oracle.h"

#include <math.h>
#include <string.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- bf16 ---------------------------------------------------------------
 * Round-to-nearest-even on the upper 16 bits, the helper the reference
 * benchmark uses on the host (benchmarks/ampere_fp8_fused_gemm_bench.cu:51-56);
 * NaN is kept quiet instead of carrying into the exponent, which is what the
 * device conversion __float2bfloat16 does. */
/* CUDA's fmaxf: a NaN operand of either kind is ignored (the other operand is returned).  glibc's fmaxf
 * returns a NaN when an operand is a SIGNALING NaN, which would reset a running maximum; all 65536 bf16
 * patterns are legal input here, so the reductions below use this form. */
static inline float max_ignoring_nan(float a, float b) {
    if (b != b) return a;
    if (a != a) return b;
    return a > b ? a : b;
}

uint16_t orc_bf16_from_f32(float v) {
    uint32_t bits = f2u(v);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x0040u);
    const uint32_t rounding = 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + rounding) >> 16);
}
/* benchmarks/ampere_fp8_fused_gemm_bench.cu:58-63 */
float orc_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

/* ---- E4M3 (OCP e4m3fn: bias 7, no inf, 0x7f NaN, max 448 = 0x7e) ---------
 * Integer restatement of include/ida_native/fp8_e4m3.hpp:31-67 for finite
 * inputs: round-to-nearest-even onto 3 mantissa bits (normals) or onto
 * multiples of 2^-9 (below 2^-6), |v| >= 448 -> 0x7e. */
static uint8_t e4m3_finite(uint32_t bits) {
    const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
    uint32_t a = bits & 0x7fffffffu;
    if (a >= 0x43e00000u) return (uint8_t)(sign | 0x7eu);          /* 448.0f */
    if (a < 0x3c800000u) {                                         /* 2^-6   */
        /* adding 2^14 leaves exactly 9 fraction bits: the sum is RNE(|v|*512)*2^-9 + 2^14 */
        const float biased = u2f(a) + 16384.0f;
        const uint32_t m = f2u(biased) & 0xfu;                     /* 0..8 */
        return (uint8_t)(sign | m);                                /* 8 == 0x08, smallest normal */
    }
    a += 0x7ffffu + ((a >> 20) & 1u);                              /* RNE at bit 20 */
    const uint32_t e = (a >> 23) - 127u + 7u;
    const uint32_t m = (a >> 20) & 7u;
    uint32_t code = (e << 3) | m;
    if (code > 0x7eu) code = 0x7eu;
    return (uint8_t)(sign | code);
}

/* include/ida_native/fp8_e4m3.hpp:31-35: nonfinite -> sign|0x7f, finite=false */
uint8_t orc_e4m3_pack(float v, int* finite) {
    const uint32_t bits = f2u(v);
    if ((bits & 0x7f800000u) == 0x7f800000u) {
        if (finite) *finite = 0;
        return (uint8_t)(((bits >> 24) & 0x80u) | 0x7fu);
    }
    if (finite) *finite = 1;
    return e4m3_finite(bits);
}

/* include/ida_native/fp8_e4m3.hpp:69-78 */
float orc_e4m3_unpack(uint8_t b) {
    const float sign = (b & 0x80u) ? -1.0f : 1.0f;
    const int e = (b >> 3) & 0xf;
    const int m = b & 7;
    if (e == 0) return sign * ldexpf((float)m, -9);
    if (e == 15 && m == 7) return NAN;
    return sign * ldexpf(1.0f + (float)m / 8.0f, e - 7);
}

/* The conversion the quantize kernels use, __nv_fp8_e4m3(float)
 * (kernels/fp8.cu:49): RNE with saturation to the largest finite value and
 * no infinities (kernels/fp8.cu:333-337), so +-inf -> +-448.  NaN -> sign|0x7f
 * (payload choice unpinned). */
uint8_t orc_e4m3_satfinite(float v) {
    const uint32_t bits = f2u(v);
    const uint32_t a = bits & 0x7fffffffu;
    const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    if (a == 0x7f800000u) return (uint8_t)(sign | 0x7eu);
    return e4m3_finite(bits);
}

/* ---- E5M2 (OCP: bias 15, inf 0x7c, NaN 0x7d..0x7f, max 57344 = 0x7b) -----
 * __nv_fp8_e5m2(float) as used at kernels/fp8.cu:59,97: RNE onto 2 mantissa
 * bits, saturate to 57344, subnormals are multiples of 2^-16. */
uint8_t orc_e5m2_satfinite(float v) {
    const uint32_t bits = f2u(v);
    uint32_t a = bits & 0x7fffffffu;
    const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    if (a >= 0x47600000u) return (uint8_t)(sign | 0x7bu);          /* 57344.0f and above, inf included */
    if (a < 0x38800000u) {                                         /* 2^-14 */
        const float biased = u2f(a) + 128.0f;                      /* 16 fraction bits remain */
        const uint32_t m = f2u(biased) & 0x7u;                     /* 0..4 */
        return (uint8_t)(sign | m);
    }
    a += 0xfffffu + ((a >> 21) & 1u);                              /* RNE at bit 21 */
    const uint32_t e = (a >> 23) - 127u + 15u;
    const uint32_t m = (a >> 21) & 3u;
    uint32_t code = (e << 2) | m;
    if (code > 0x7bu) code = 0x7bu;
    return (uint8_t)(sign | code);
}

float orc_e5m2_unpack(uint8_t b) {
    const float sign = (b & 0x80u) ? -1.0f : 1.0f;
    const int e = (b >> 2) & 0x1f;
    const int m = b & 3;
    if (e == 0) return sign * ldexpf((float)m, -16);
    if (e == 31) return m == 0 ? sign * INFINITY : NAN;
    return sign * ldexpf(1.0f + (float)m / 4.0f, e - 15);
}

void orc_bf16_from_f32_n(const float* in, uint16_t* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_from_f32(in[i]); }
void orc_bf16_to_f32_n(const uint16_t* in, float* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]); }
void orc_e4m3_pack_n(const float* in, uint8_t* out, uint8_t* finite, size_t n) {
    for (size_t i = 0; i < n; ++i) { int f; out[i] = orc_e4m3_pack(in[i], &f); if (finite) finite[i] = (uint8_t)f; }
}
void orc_e4m3_satfinite_n(const float* in, uint8_t* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_e4m3_satfinite(in[i]); }
void orc_e5m2_satfinite_n(const float* in, uint8_t* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_e5m2_satfinite(in[i]); }
void orc_e4m3_unpack_n(const uint8_t* in, float* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_e4m3_unpack(in[i]); }
void orc_e5m2_unpack_n(const uint8_t* in, float* out, size_t n) { for (size_t i = 0; i < n; ++i) out[i] = orc_e5m2_unpack(in[i]); }

/* ---- per-tensor quantize family ---------------------------------------- */

/* kernels/fp8.cu:22-32,250-253: result starts from 0 (the wrapper zeroes it),
 * fmaxf ignores NaN operands. */
void orc_amax_bf16(const uint16_t* x, size_t n, float* amax) {
    float local = 0.0f;
    for (size_t i = 0; i < n; ++i) local = max_ignoring_nan(local, fabsf(orc_bf16_to_f32(x[i])));
    *amax = local;
}

/* kernels/fp8.cu:34-40 */
void orc_scale_from_amax(const float* amax, float fp8_max, float* scale, float* descale) {
    const float a = fmaxf(*amax, 1e-12f);
    *scale = fp8_max / a;
    *descale = a / fp8_max;
}

/* kernels/fp8.cu:42-50 */
void orc_quantize_e4m3(const uint16_t* x, uint8_t* out, const float* scale, size_t n) {
    const float s = *scale;
    for (size_t i = 0; i < n; ++i) out[i] = orc_e4m3_satfinite(orc_bf16_to_f32(x[i]) * s);
}
/* kernels/fp8.cu:52-60 */
void orc_quantize_e5m2(const uint16_t* x, uint8_t* out, const float* scale, size_t n) {
    const float s = *scale;
    for (size_t i = 0; i < n; ++i) out[i] = orc_e5m2_satfinite(orc_bf16_to_f32(x[i]) * s);
}

/* kernels/fp8.cu:67-84: amax of the UNSCALED input is max-combined into *amax
 * (integer atomicMax on non-negative float bits == fmaxf), the caller zeroes it. */
void orc_quantize_e4m3_record(const uint16_t* x, uint8_t* out, const float* scale, float* amax, size_t n) {
    const float s = *scale;
    float local = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        const float v = orc_bf16_to_f32(x[i]);
        local = max_ignoring_nan(local, fabsf(v));
        out[i] = orc_e4m3_satfinite(v * s);
    }
    if ((int32_t)f2u(local) > (int32_t)f2u(*amax)) *amax = local;
}
/* kernels/fp8.cu:86-103 */
void orc_quantize_e5m2_record(const uint16_t* x, uint8_t* out, const float* scale, float* amax, size_t n) {
    const float s = *scale;
    float local = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        const float v = orc_bf16_to_f32(x[i]);
        local = max_ignoring_nan(local, fabsf(v));
        out[i] = orc_e5m2_satfinite(v * s);
    }
    if ((int32_t)f2u(local) > (int32_t)f2u(*amax)) *amax = local;
}

/* kernels/fp8.cu:105-142 */
void orc_update_delayed_scale(const float* amax, float fp8_max, float* scale, float* descale,
                              float* history, int history_len, int* cursor_p, int* count_p) {
    const float a = fmaxf(*amax, 1e-12f);
    int cursor = *cursor_p;
    int count = *count_p;
    if (history_len <= 0) {
        *scale = fp8_max / a;
        *descale = a / fp8_max;
        return;
    }
    if (cursor < 0 || cursor >= history_len) cursor = 0;
    history[cursor] = a;
    cursor = (cursor + 1) % history_len;
    if (count < history_len) ++count;
    float hist_max = history[0];
    for (int i = 1; i < count; ++i) hist_max = fmaxf(hist_max, history[i]);
    hist_max = fmaxf(hist_max, 1e-12f);
    *cursor_p = cursor;
    *count_p = count;
    *scale = fp8_max / hist_max;
    *descale = hist_max / fp8_max;
}

/* kernels/fp8.cu:230-243: w[K,N] -> out[N,K] */
void orc_quantize_transpose_e4m3(const uint16_t* w, uint8_t* out, const float* scale, int K, int N) {
    const float s = *scale;
    for (int k = 0; k < K; ++k)
        for (int c = 0; c < N; ++c)
            out[(size_t)c * K + k] = orc_e4m3_satfinite(orc_bf16_to_f32(w[(size_t)k * N + c]) * s);
}

/* kernels/fp8.cu:151-227: in[K,N] -> act8[K,N] and snap[N,K] */
void orc_quant_and_transpose_e4m3(const uint16_t* in, uint8_t* act8, uint8_t* snap,
                                  const float* scale, int K, int N) {
    const float s = *scale;
    for (int k = 0; k < K; ++k)
        for (int c = 0; c < N; ++c) {
            const uint8_t q = orc_e4m3_satfinite(orc_bf16_to_f32(in[(size_t)k * N + c]) * s);
            act8[(size_t)k * N + c] = q;
            snap[(size_t)c * K + k] = q;
        }
}

/* src/trainer.cu:1392-1448: in[rows,cols] -> out[cols,rows] */
void orc_transpose_u8(const uint8_t* in, uint8_t* out, int rows, int cols) {
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) out[(size_t)c * rows + r] = in[(size_t)r * cols + c];
}

/* kernels/fp8.cu:342-356 */
void orc_clip_probe(const float* amax, const float* scale, float fp8_max, float* stats) {
    const float a = *amax;
    const float s = *scale;
    stats[2] += 1.0f;
    if (fp8_max > 0.0f && s > 0.0f) {
        const float ratio = a * s / fp8_max;
        if (ratio > 1.0f) {
            stats[0] += 1.0f;
            if (ratio > stats[1]) stats[1] = ratio;
        }
    }
}

/* kernels/fp8.cu:374-387 (counts are exact integers; compared below 2^24) */
void orc_elem_clip_count(const uint16_t* x, const float* scale, float fp8_max, size_t n, float* out) {
    const float s = *scale;
    size_t clipped = 0;
    for (size_t i = 0; i < n; ++i)
        if (fabsf(orc_bf16_to_f32(x[i])) * s > fp8_max) ++clipped;
    out[0] += (float)clipped;
    out[1] += (float)n;
}

/* kernels/fp8.cu:422-446,491-503.  bad_count is used by the caller as a
 * predicate only (src/trainer.cu:3397-3408); the reference's numeric value
 * depends on its 32-lane launch geometry.  Here it is the number of nonfinite
 * inputs plus the number of nonfinite packed products. */
static void raw_stats(const uint16_t* x, size_t n, float* amax, int* bad) {
    float local = 0.0f;
    int nbad = 0;
    for (size_t i = 0; i < n; ++i) {
        const float v = orc_bf16_to_f32(x[i]);
        if (!isfinite(v)) ++nbad; else local = fmaxf(local, fabsf(v));
    }
    *amax = local;
    *bad = nbad;
}
void orc_pack_bf16_e4m3_raw(const uint16_t* x, uint8_t* out, float* amax, float* scale,
                            float* descale, int* bad_count, size_t n) {
    raw_stats(x, n, amax, bad_count);
    orc_scale_from_amax(amax, 448.0f, scale, descale);
    const float s = *scale;
    for (size_t i = 0; i < n; ++i) {
        int fin;
        out[i] = orc_e4m3_pack(orc_bf16_to_f32(x[i]) * s, &fin);   /* kernels/fp8.cu:448-459 */
        if (!fin) ++*bad_count;
    }
}
/* kernels/fp8.cu:473-489,505-522 */
void orc_pack_bf16_e4m3_raw_and_dequant(const uint16_t* x, uint8_t* out, uint16_t* dequant,
                                        float* amax, float* scale, float* descale,
                                        int* bad_count, size_t n) {
    raw_stats(x, n, amax, bad_count);
    orc_scale_from_amax(amax, 448.0f, scale, descale);
    const float s = *scale, d = *descale;
    for (size_t i = 0; i < n; ++i) {
        int fin;
        out[i] = orc_e4m3_pack(orc_bf16_to_f32(x[i]) * s, &fin);
        dequant[i] = orc_bf16_from_f32(orc_e4m3_unpack(out[i]) * d);
        if (!fin) ++*bad_count;
    }
}
/* kernels/fp8.cu:461-470 */
void orc_unpack_e4m3_raw_bf16(const uint8_t* in, const float* descale, uint16_t* out, size_t n) {
    const float d = *descale;
    for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_from_f32(orc_e4m3_unpack(in[i]) * d);
}

/* src/trainer.cu:3789-3795 */
void orc_calib_minmax_update(const float* amax, float* cmin, float* cmax) {
    const float a = fmaxf(*amax, 1e-12f);
    *cmin = fminf(*cmin, a);
    *cmax = fmaxf(*cmax, a);
}

/* ---- scale-group extensions ---------------------------------------------
 * The reference scales per tensor only (kernels/fp8.cu:13-16).  The grouped
 * forms apply the identical formula (kernels/fp8.cu:37-39,49) to a smaller
 * group: amax over the group, scale = fp8_max / max(amax,1e-12),
 * descale = max(amax,1e-12) / fp8_max, code = cvt(x * scale). */
void orc_amax_f32(const float* x, size_t n, float* amax) {
    float local = 0.0f;
    for (size_t i = 0; i < n; ++i) local = max_ignoring_nan(local, fabsf(x[i]));
    *amax = local;
}
void orc_quantize_f32_e4m3(const float* x, uint8_t* out, const float* scale, size_t n) {
    const float s = *scale;
    for (size_t i = 0; i < n; ++i) out[i] = orc_e4m3_satfinite(x[i] * s);
}

void orc_quantize_rows(const uint16_t* x, int rows, int K, int is_e5m2,
                       uint8_t* out, float* scale, float* descale) {
    const float fmax_ = is_e5m2 ? ORC_E5M2_MAX : ORC_E4M3_MAX;
    for (int r = 0; r < rows; ++r) {
        float amax;
        orc_amax_bf16(x + (size_t)r * K, (size_t)K, &amax);
        orc_scale_from_amax(&amax, fmax_, &scale[r], &descale[r]);
        if (is_e5m2) orc_quantize_e5m2(x + (size_t)r * K, out + (size_t)r * K, &scale[r], (size_t)K);
        else         orc_quantize_e4m3(x + (size_t)r * K, out + (size_t)r * K, &scale[r], (size_t)K);
    }
}

void orc_quantize_block_1x128(const uint16_t* x, int rows, int K,
                              uint8_t* out, float* scale, float* descale) {
    const int kb = (K + 127) / 128;
    for (int r = 0; r < rows; ++r)
        for (int b = 0; b < kb; ++b) {
            const int k0 = b * 128, len = (K - k0 < 128) ? K - k0 : 128;
            const size_t off = (size_t)r * K + k0, si = (size_t)r * kb + b;
            float amax;
            orc_amax_bf16(x + off, (size_t)len, &amax);
            orc_scale_from_amax(&amax, ORC_E4M3_MAX, &scale[si], &descale[si]);
            orc_quantize_e4m3(x + off, out + off, &scale[si], (size_t)len);
        }
}

void orc_quantize_block_128x128(const uint16_t* x, int rows, int K,
                                uint8_t* out, float* scale, float* descale) {
    const int kb = (K + 127) / 128, rb = (rows + 127) / 128;
    for (int br = 0; br < rb; ++br)
        for (int b = 0; b < kb; ++b) {
            const int r0 = br * 128, r1 = (r0 + 128 < rows) ? r0 + 128 : rows;
            const int k0 = b * 128, len = (K - k0 < 128) ? K - k0 : 128;
            const size_t si = (size_t)br * kb + b;
            float amax = 0.0f;
            for (int r = r0; r < r1; ++r) {
                float a;
                orc_amax_bf16(x + (size_t)r * K + k0, (size_t)len, &a);
                amax = max_ignoring_nan(amax, a);
            }
            orc_scale_from_amax(&amax, ORC_E4M3_MAX, &scale[si], &descale[si]);
            for (int r = r0; r < r1; ++r)
                orc_quantize_e4m3(x + (size_t)r * K + k0, out + (size_t)r * K + k0, &scale[si], (size_t)len);
        }
}

/* ---- elementwise epilogue ops -------------------------------------------
 * kernels/activations.cu:11-40.  The exponential is orc_expf, this build's
 * definition of the device expf (see cf_oracle.h). */
static float stable_sigmoid(float x) {
    if (x >= 0.0f) return 1.0f / (1.0f + orc_expf(-x));
    const float e = orc_expf(x);
    return e / (1.0f + e);
}
void orc_swiglu_forward(const uint16_t* gate, const uint16_t* up, uint16_t* out, int n) {
    for (int i = 0; i < n; ++i) {
        const float g = orc_bf16_to_f32(gate[i]);
        const float u = orc_bf16_to_f32(up[i]);
        const float silu = g * stable_sigmoid(g);
        out[i] = orc_bf16_from_f32(silu * u);
    }
}

/* kernels/activations.cu:23-26 (silu_derivative), :42-58 (k_swiglu_backward): the products are taken left to right,
 * grad_gate = bf16((grad * up) * silu'(gate)), grad_up = bf16(grad * silu(gate)). */
void orc_swiglu_backward(const uint16_t* grad_out, const uint16_t* gate, const uint16_t* up,
                         uint16_t* grad_gate, uint16_t* grad_up, int n) {
    for (int i = 0; i < n; ++i) {
        const float g = orc_bf16_to_f32(gate[i]);
        const float u = orc_bf16_to_f32(up[i]);
        const float d = orc_bf16_to_f32(grad_out[i]);
        const float sg = stable_sigmoid(g);
        const float dsilu = sg * (1.0f + g * (1.0f - sg));
        const float silu = g * sg;
        grad_gate[i] = orc_bf16_from_f32((d * u) * dsilu);
        grad_up[i] = orc_bf16_from_f32(d * silu);
    }
}

/* kernels/moe.cu:335-348 (k_col_sum_strided_bf16): one fp32 running sum per column over the rows in ascending
 * order, started at zero and then added to what the accumulator holds. */
void orc_col_sum_strided_bf16(const uint16_t* in, float* out_accum, int rows, int cols, int row_stride, int base) {
    for (int c = 0; c < cols; ++c) {
        float acc = 0.0f;
        for (int r = 0; r < rows; ++r) acc += orc_bf16_to_f32(in[(size_t)r * row_stride + base + c]);
        out_accum[c] += acc;
    }
}

/* kernels/moe.cu:325-334 */
void orc_bias_add_strided_bf16(uint16_t* inout, const uint16_t* bias,
                               int rows, int cols, int row_stride, int base) {
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) {
            uint16_t* p = inout + (size_t)r * row_stride + base + c;
            *p = orc_bf16_from_f32(orc_bf16_to_f32(*p) + orc_bf16_to_f32(bias[c]));
        }
}
