// Producers of the quantizer's input, fused with it: RMSNorm forward, the absolute-ceiling activation
// row clip, and the per-row / recording FP8 quantize, in one pass over the activations.
//
// The reference runs rmsnorm_forward (kernels/rmsnorm.cu:13-54,101-108), act_row_clip
// (src/trainer.cu:3822-3842,3940-3991) and the quantize (kernels/fp8.cu:67-103) as four launches that read the
// row from HBM four times and write it twice.  Here one workgroup owns one row: the row is loaded once into
// LDS, every later step (two reductions, normalise, clip, amax, convert) works on the LDS copy, and HBM sees
// 2 B read + (2 B normalised row, if asked for) + 1 B fp8 written per element.
//
// The bf16 results depend on the order of the fp32 sums, so both reductions follow the reference's trees
// exactly: per-thread partials over the elements t, t + T, ... (one fused multiply-add each, as nvcc contracts
// `s += v * v`), a 32-lane xor butterfly, then the second stage over the 32-lane leaders (a butterfly in
// rmsnorm, a sequential sum in the clip).
#include "common.hpp"

namespace cf {
namespace {

constexpr int kNormMaxThreads = 512;      // kernels/rmsnorm.cu:106
constexpr int kClipThreads = 256;         // src/trainer.cu:3989
constexpr int kNormMaxH = 16384;          // the row lives in LDS as bf16

enum { Q_NONE = 0, Q_ROWS = 1, Q_RECORD = 2 };

struct NormArgs {
    const uint16_t* x;        // [rows, H] bf16
    const uint16_t* weight;   // [H] bf16 (NORM only)
    uint16_t* normed;         // [rows, H] bf16 or null
    float* rms;               // [rows] or null
    float* normsq;            // [rows] or null: the clip's row sums of squares
    uint8_t* q;               // [rows, H] fp8
    float* row_scale;         // Q_ROWS: [rows]
    float* row_descale;
    const float* qscale;      // Q_RECORD: the scale to quantize with
    float* amax;              // Q_RECORD: running maximum, raised atomically
    int H;
    float eps;
    float ceiling;            // <= 0: no clip
};

__device__ __forceinline__ float butterfly32(float v) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// VEC: H % 8 == 0 and every row pointer 16-byte aligned (fp8 rows 8-byte): the row moves as 8-element chunks,
// chunk c of a row belonging to thread c % T.  Otherwise single elements with the same ownership rule.
template <bool NORM, int QMODE, bool E5M2, bool VEC>   // QMODE != Q_NONE only with NORM
__global__ __launch_bounds__(kNormMaxThreads) void k_norm_clip_quant(const NormArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];      // the row, H bf16
    __shared__ float sh[40];
    const int t = threadIdx.x, T = blockDim.x, H = p.H;
    const size_t row = blockIdx.x;
    const uint16_t* xr = p.x + row * H;
    constexpr int CH = VEC ? 8 : 1;
    const int nchunks = H / CH;

    for (int c = t; c < nchunks; c += T) {
        if constexpr (VEC) reinterpret_cast<uint4*>(xs)[c] = reinterpret_cast<const uint4*>(xr)[c];
        else xs[c] = xr[c];
    }
    __syncthreads();

    float local_amax = 0.0f;
    if constexpr (NORM) {
        // mean square: kernels/rmsnorm.cu:24-45
        float ms = 0.0f;
        for (int h = t; h < H; h += T) {
            const float v = bf16_to_f32(xs[h]);
            ms = __builtin_fmaf(v, v, ms);
        }
        ms = butterfly32(ms);
        if ((t & 31) == 0) sh[t >> 5] = ms;
        __syncthreads();
        if (t < 32) {
            float l = (t < (T + 31) / 32) ? sh[t] : 0.0f;
            l = butterfly32(l);
            if (t == 0) sh[32] = l;
        }
        __syncthreads();
        const float rms_val = sqrtf(sh[32] / static_cast<float>(H) + p.eps);
        if (t == 0 && p.rms) p.rms[row] = rms_val;
        const float inv_rms = 1.0f / rms_val;
        // normalise in place: kernels/rmsnorm.cu:48-52
        for (int c = t; c < nchunks; c += T) {
            if constexpr (VEC) {
                const uint4 xv = reinterpret_cast<const uint4*>(xs)[c];
                const uint4 wv = reinterpret_cast<const uint4*>(p.weight)[c];
                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lo = (bf16_lo(xw[i]) * inv_rms) * bf16_lo(ww[i]);
                    const float hi = (bf16_hi(xw[i]) * inv_rms) * bf16_hi(ww[i]);
                    o[i] = pack_bf16x2(lo, hi);
                    local_amax = fmaxf(local_amax, fmaxf(fabsf(bf16_lo(o[i])), fabsf(bf16_hi(o[i]))));
                }
                reinterpret_cast<uint4*>(xs)[c] = make_uint4(o[0], o[1], o[2], o[3]);
            } else {
                const uint16_t o = f32_to_bf16((bf16_to_f32(xs[c]) * inv_rms) * bf16_to_f32(p.weight[c]));
                local_amax = fmaxf(local_amax, fabsf(bf16_to_f32(o)));
                xs[c] = o;
            }
        }
    }

    if (p.ceiling > 0.0f) {
        // row sum of squares with the clip kernel's tree: src/trainer.cu:3822-3842
        __syncthreads();
        if (t < kClipThreads) {
            float s = 0.0f;
            for (int c = t; c < H; c += kClipThreads) {
                const float v = bf16_to_f32(xs[c]);
                s = __builtin_fmaf(v, v, s);
            }
            s = butterfly32(s);
            if ((t & 31) == 0) sh[t >> 5] = s;
        }
        __syncthreads();
        float total = 0.0f;
        const int leaders = min(T, kClipThreads) / 32;     // absent leaders would add +0
        for (int w = 0; w < leaders; ++w) total += sh[w];
        if (t == 0 && p.normsq) p.normsq[row] = total;
        // src/trainer.cu:3946-3957
        const float norm = sqrtf(total);
        if (!(norm <= p.ceiling)) {
            const float scalef = p.ceiling / norm;
            local_amax = 0.0f;
            for (int c = t; c < nchunks; c += T) {
                if constexpr (VEC) {
                    const uint4 xv = reinterpret_cast<const uint4*>(xs)[c];
                    const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
                    uint32_t o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        o[i] = pack_bf16x2(bf16_lo(xw[i]) * scalef, bf16_hi(xw[i]) * scalef);
                        local_amax = fmaxf(local_amax, fmaxf(fabsf(bf16_lo(o[i])), fabsf(bf16_hi(o[i]))));
                    }
                    reinterpret_cast<uint4*>(xs)[c] = make_uint4(o[0], o[1], o[2], o[3]);
                } else {
                    const uint16_t o = f32_to_bf16(bf16_to_f32(xs[c]) * scalef);
                    local_amax = fmaxf(local_amax, fabsf(bf16_to_f32(o)));
                    xs[c] = o;
                }
            }
        }
    }

    // the row's scale: kernels/fp8.cu:34-40 on the row maximum, or the caller's scale with the maximum recorded
    float qs = 0.0f;
    if constexpr (QMODE != Q_NONE) {
        // reduced over 32-lane groups: T may end in half a wavefront
        float m = local_amax;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, kWave));
        __syncthreads();                                   // sh is free again
        if ((t & 31) == 0) sh[t >> 5] = m;
        __syncthreads();
        m = sh[0];
        for (int w = 1; w < T / 32; ++w) m = fmaxf(m, sh[w]);
        constexpr float fmax_ = E5M2 ? 57344.0f : 448.0f;
        if constexpr (QMODE == Q_ROWS) {
            const float a = fmaxf(m, 1e-12f);
            qs = fmax_ / a;
            if (t == 0) { p.row_scale[row] = qs; p.row_descale[row] = a / fmax_; }
        } else {
            qs = *p.qscale;
            if (t == 0) atomic_max_nonneg(p.amax, m);
        }
    }

    // out: each thread stores the chunks it owns (its own LDS writes need no barrier)
    uint16_t* nr = p.normed ? p.normed + row * H : nullptr;
    uint8_t* qr = (QMODE != Q_NONE) ? p.q + row * H : nullptr;
    for (int c = t; c < nchunks; c += T) {
        if constexpr (VEC) {
            const uint4 v = reinterpret_cast<const uint4*>(xs)[c];
            if (nr) reinterpret_cast<uint4*>(nr)[c] = v;
            if constexpr (QMODE != Q_NONE) {
                uint2 o;
                o.x = cvt4_fp8<E5M2>(bf16_lo(v.x) * qs, bf16_hi(v.x) * qs, bf16_lo(v.y) * qs, bf16_hi(v.y) * qs);
                o.y = cvt4_fp8<E5M2>(bf16_lo(v.z) * qs, bf16_hi(v.z) * qs, bf16_lo(v.w) * qs, bf16_hi(v.w) * qs);
                reinterpret_cast<uint2*>(qr)[c] = o;
            }
        } else {
            const uint16_t v = xs[c];
            if (nr) nr[c] = v;
            if constexpr (QMODE != Q_NONE) qr[c] = cvt1_fp8<E5M2>(bf16_to_f32(v) * qs);
        }
    }
}

template <bool NORM, int QMODE>
int launch_norm(const NormArgs& p, int rows, bool e5m2, hipStream_t st) {
    const int H = p.H;
    const int T = H < kNormMaxThreads ? H : kNormMaxThreads;
    bool vec = H % 8 == 0 && aligned16(p.x) && (!p.normed || aligned16(p.normed)) && (!NORM || aligned16(p.weight));
    if (QMODE != Q_NONE && (reinterpret_cast<uintptr_t>(p.q) & 7u) != 0) vec = false;
    const size_t lds = static_cast<size_t>(H) * 2;
    auto go = [&](auto kernel) {
        kernel<<<rows, T, lds, st>>>(p);
        return launch_status();
    };
    if (vec) return e5m2 ? go(k_norm_clip_quant<NORM, QMODE, true, true>) : go(k_norm_clip_quant<NORM, QMODE, false, true>);
    return e5m2 ? go(k_norm_clip_quant<NORM, QMODE, true, false>) : go(k_norm_clip_quant<NORM, QMODE, false, false>);
}

// 0: run, 1: nothing to do, < 0: error
int check_shape(int rows, int H, bool norm) {
    if (rows < 0 || H < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || H == 0) return 1;
    if (H > kNormMaxH) return CF_ERR_UNSUPPORTED;
    // the reference's reduction is defined for whole 32-lane groups only (full-mask shuffles)
    if (norm && (H < kNormMaxThreads ? H : kNormMaxThreads) % 32 != 0) return CF_ERR_UNSUPPORTED;
    if (!norm && H < kClipThreads && H % 32 != 0) return CF_ERR_UNSUPPORTED;
    return 0;
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_rmsnorm_forward(const uint16_t* d_x, const uint16_t* d_scale, uint16_t* d_out, float* d_rms, int rows,
                       int H, float eps, cf_stream_t stream) {
    const int chk = check_shape(rows, H, true);
    if (chk != 0) return chk < 0 ? chk : CF_OK;
    if (!d_x || !d_scale || !d_out) return CF_ERR_INVALID_ARG;
    NormArgs p{};
    p.x = d_x; p.weight = d_scale; p.normed = d_out; p.rms = d_rms; p.H = H; p.eps = eps; p.ceiling = 0.0f;
    return launch_norm<true, Q_NONE>(p, rows, false, as_stream(stream));
}

int cf_act_row_clip_abs(uint16_t* d_x, int rows, int cols, float ceiling, float* d_normsq, cf_stream_t stream) {
    const int chk = check_shape(rows, cols, false);
    if (chk != 0) return chk < 0 ? chk : CF_OK;
    if (!(ceiling > 0.0f)) return CF_OK;             // src/trainer.cu:3974
    if (!d_x) return CF_ERR_INVALID_ARG;
    NormArgs p{};
    p.x = d_x; p.normed = d_x; p.normsq = d_normsq; p.H = cols; p.ceiling = ceiling;
    // fewer than 256 columns: the clip kernel's threads beyond the row hold zero partials
    return launch_norm<false, Q_NONE>(p, rows, false, as_stream(stream));
}

int cf_rmsnorm_clip_quantize_rows(const uint16_t* d_x, const uint16_t* d_scale, int rows, int H, float eps,
                                  float ceiling, int is_e5m2, uint16_t* d_normed, float* d_rms, void* d_q,
                                  float* d_row_scale, float* d_row_descale, cf_stream_t stream) {
    const int chk = check_shape(rows, H, true);
    if (chk != 0) return chk < 0 ? chk : CF_OK;
    if (!d_x || !d_scale || !d_q || !d_row_scale || !d_row_descale) return CF_ERR_INVALID_ARG;
    NormArgs p{};
    p.x = d_x; p.weight = d_scale; p.normed = d_normed; p.rms = d_rms; p.q = static_cast<uint8_t*>(d_q);
    p.row_scale = d_row_scale; p.row_descale = d_row_descale; p.H = H; p.eps = eps; p.ceiling = ceiling;
    return launch_norm<true, Q_ROWS>(p, rows, is_e5m2 != 0, as_stream(stream));
}

int cf_rmsnorm_clip_quantize_record(const uint16_t* d_x, const uint16_t* d_scale, int rows, int H, float eps,
                                    float ceiling, int is_e5m2, uint16_t* d_normed, float* d_rms, void* d_q,
                                    const float* d_qscale, float* d_amax, cf_stream_t stream) {
    const int chk = check_shape(rows, H, true);
    if (chk != 0) return chk < 0 ? chk : CF_OK;
    if (!d_x || !d_scale || !d_q || !d_qscale || !d_amax) return CF_ERR_INVALID_ARG;
    NormArgs p{};
    p.x = d_x; p.weight = d_scale; p.normed = d_normed; p.rms = d_rms; p.q = static_cast<uint8_t*>(d_q);
    p.qscale = d_qscale; p.amax = d_amax; p.H = H; p.eps = eps; p.ceiling = ceiling;
    return launch_norm<true, Q_RECORD>(p, rows, is_e5m2 != 0, as_stream(stream));
}

}  // extern "C"
