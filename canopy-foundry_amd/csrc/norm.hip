// Producers of the quantizer's input, fused with it: RMSNorm forward, the absolute-ceiling activation
// row clip, and the per-row / recording FP8 quantize, in one pass over the activations.
//
// The reference runs rmsnorm_forward (kernels/rmsnorm.cu:13-54,101-108), act_row_clip
// (src/trainer.cu:3822-3842,3940-3991) and the quantize (kernels/fp8.cu:67-103) as four launches that read the
// row from HBM four times and write it twice.  Here a row is loaded once, every later step (two reductions,
// normalise, clip, amax, convert) works on that copy, and HBM sees 2 B read + (2 B normalised row, if asked
// for) + 1 B fp8 written per element.
//
// The bf16 results depend on the order of the fp32 sums, so both reductions follow the reference's trees
// exactly: per-thread partials over the elements t, t + T, ... (one fused multiply-add each, as nvcc contracts
// `s += v * v`), a 32-lane xor butterfly, then the second stage over the 32-lane leaders (a butterfly in
// rmsnorm, a sequential sum in the clip).
//
// Two kernels.  k_norm_row_wave (H a multiple of 512 up to 8192, aligned rows): one wavefront owns a row and
// keeps it in registers; lane l holds the elements 8l..8l+7 of every 512-element stripe, which are exactly
// the elements of the reference's threads 8l..8l+7, so the per-thread partial sums need no communication and the
// butterflies become two lane shuffles plus in-lane adds.  No LDS, no barriers.  k_norm_clip_quant (any other
// supported shape): one workgroup per row with the row in LDS and the reference's thread count.
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

// ---- one wavefront per row --------------------------------------------------------------------
// J = H / 512 stripes.  Lane l holds chunk j = elements 512 j + 8 l .. + 7 as four packed dwords.
__device__ __forceinline__ float bf16_at(const uint4& v, int i) {
    const uint32_t w = (i < 2) ? v.x : (i < 4) ? v.y : (i < 6) ? v.z : v.w;
    return (i & 1) ? bf16_hi(w) : bf16_lo(w);
}
// Eight per-lane partials of the reference's threads 8 l + i -> the sum over the 32-thread group that the four
// lanes l & ~3 .. l | 3 make up, in the order of the xor butterfly (offsets 16, 8 across lanes; 4, 2, 1 in-lane).
__device__ __forceinline__ float group32_sum(float (&part)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) part[i] += __shfl_xor(part[i], 2, kWave);
#pragma unroll
    for (int i = 0; i < 8; ++i) part[i] += __shfl_xor(part[i], 1, kWave);
    const float a0 = part[0] + part[4], a1 = part[1] + part[5], a2 = part[2] + part[6], a3 = part[3] + part[7];
    const float b0 = a0 + a2, b1 = a1 + a3;
    return b0 + b1;
}

template <int J, bool NORM, int QMODE, bool E5M2>   // QMODE != Q_NONE only with NORM
__global__ __launch_bounds__(256) void k_norm_row_wave(const NormArgs p, int rows) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;                                  // whole wavefronts
    constexpr int H = J * 512;
    const size_t base = static_cast<size_t>(row) * H + 8 * lane;
    uint4 v[J];
#pragma unroll
    for (int j = 0; j < J; ++j) v[j] = *reinterpret_cast<const uint4*>(p.x + base + 512 * j);

    auto rewrite = [&](int j, auto f) {      // v[j][i] <- bf16(f(value, i))
        // The words are hidden from common-subexpression elimination: otherwise the fp32 values unpacked for the sum
        // of squares stay live until here (64 more registers per lane at H = 4096); unpacking again is one
        // instruction per element.
        uint32_t w[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
        asm volatile("" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]));
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = pack_bf16x2_hw(f(bf16_lo(w[k]), 2 * k), f(bf16_hi(w[k]), 2 * k + 1));
        v[j] = make_uint4(o[0], o[1], o[2], o[3]);
    };

    if constexpr (NORM) {
        // kernels/rmsnorm.cu:24-41: 512 threads, 16 groups of 32; the second butterfly runs over 32 slots of which
        // the upper 16 are zero (adding +0 changes nothing), so it is four exchanges across the 16 groups
        float part[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = bf16_at(v[j], i);
                part[i] = __builtin_fmaf(x, x, part[i]);
            }
        float total = group32_sum(part);
        total += __shfl_xor(total, 32, kWave);
        total += __shfl_xor(total, 16, kWave);
        total += __shfl_xor(total, 8, kWave);
        total += __shfl_xor(total, 4, kWave);
        const float rms_val = sqrtf(total / static_cast<float>(H) + p.eps);      // :44-45
        if (lane == 0 && p.rms) p.rms[row] = rms_val;
        const float inv_rms = 1.0f / rms_val;
#pragma unroll
        for (int j = 0; j < J; ++j) {                                            // :48-52
            const uint4 w = *reinterpret_cast<const uint4*>(p.weight + 8 * lane + 512 * j);
            rewrite(j, [&](float x, int i) { return (x * inv_rms) * bf16_at(w, i); });
        }
    }

    if (p.ceiling > 0.0f) {
        // src/trainer.cu:3822-3842: 256 threads; thread 8 (l % 32) + i walks the row with stride 256, which
        // alternates between the stripe of lane l % 32 and that of lane l % 32 + 32.  The lower lanes walk the
        // chains i = 0..3, the upper lanes i = 4..7, each with its own half chunk and the partner's.
        float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const bool upper = lane >= 32;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const uint32_t t0 = __shfl_xor(upper ? v[j].x : v[j].z, 32, kWave);
            const uint32_t t1 = __shfl_xor(upper ? v[j].y : v[j].w, 32, kWave);
            const uint32_t first[2] = {upper ? t0 : v[j].x, upper ? t1 : v[j].y};       // the lower lane's half
            const uint32_t second[2] = {upper ? v[j].z : t0, upper ? v[j].w : t1};      // the upper lane's half
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float x = (i & 1) ? bf16_hi(first[i >> 1]) : bf16_lo(first[i >> 1]);
                s[i] = __builtin_fmaf(x, x, s[i]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float x = (i & 1) ? bf16_hi(second[i >> 1]) : bf16_lo(second[i >> 1]);
                s[i] = __builtin_fmaf(x, x, s[i]);
            }
        }
        // butterfly of the 32-thread group 8 (l % 4) + i: offsets 16 and 8 across lanes, 4 across the halves, 2 and 1 in-lane
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += __shfl_xor(s[i], 2, kWave);
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += __shfl_xor(s[i], 1, kWave);
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += __shfl_xor(s[i], 32, kWave);
        const float leader = (s[0] + s[2]) + (s[1] + s[3]);          // group g of 8 sits in lanes 4 g .. 4 g + 3
        float total = 0.0f;
#pragma unroll
        for (int g = 0; g < 8; ++g) total += __shfl(leader, 4 * g, kWave);          // :3837-3839
        if (lane == 0 && p.normsq) p.normsq[row] = total;
        const float norm = sqrtf(total);                                        // :3946-3957
        if (!(norm <= p.ceiling)) {
            const float scalef = p.ceiling / norm;
#pragma unroll
            for (int j = 0; j < J; ++j) rewrite(j, [&](float x, int) { return x * scalef; });
        }
    }

    float qs = 0.0f;
    bool finite = true;
    if constexpr (QMODE != Q_NONE) {
        uint32_t acc = 0;
#pragma unroll
        for (int j = 0; j < J; ++j) acc = pk_absmax(pk_absmax(pk_absmax(pk_absmax(acc, v[j].x), v[j].y), v[j].z), v[j].w);
        const int mbits = wave_absmax_bits(acc);
        finite = mbits < 0x7f80;
        float m = __uint_as_float(static_cast<uint32_t>(mbits) << 16);
        if (!finite) {
            // the maximum that ignores NaNs, as a float maximum does
            float local = 0.0f;
#pragma unroll
            for (int j = 0; j < J; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i) local = fmaxf(local, fabsf(bf16_at(v[j], i)));
            m = wave_max(local);
        }
        constexpr float fmax_ = E5M2 ? 57344.0f : 448.0f;
        if constexpr (QMODE == Q_ROWS) {
            const float a = fmaxf(m, 1e-12f);
            qs = fmax_ / a;
            if (lane == 0) { p.row_scale[row] = qs; p.row_descale[row] = a / fmax_; }
        } else {
            qs = *p.qscale;
            if (lane == 0) atomic_max_nonneg(p.amax, m);
            finite = finite && fabsf(qs) < __uint_as_float(0x7f800000u);     // 0 x inf would make a NaN
        }
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        if (p.normed) store_stream16(p.normed + base + 512 * j, v[j]);
        if constexpr (QMODE != Q_NONE) {
            uint2 o;
            if (finite) {     // every product is finite: no NaN code to restore
                o.x = cvt4_fp8_finite<E5M2>(bf16_lo(v[j].x) * qs, bf16_hi(v[j].x) * qs, bf16_lo(v[j].y) * qs, bf16_hi(v[j].y) * qs);
                o.y = cvt4_fp8_finite<E5M2>(bf16_lo(v[j].z) * qs, bf16_hi(v[j].z) * qs, bf16_lo(v[j].w) * qs, bf16_hi(v[j].w) * qs);
            } else {
                o.x = cvt4_fp8<E5M2>(bf16_lo(v[j].x) * qs, bf16_hi(v[j].x) * qs, bf16_lo(v[j].y) * qs, bf16_hi(v[j].y) * qs);
                o.y = cvt4_fp8<E5M2>(bf16_lo(v[j].z) * qs, bf16_hi(v[j].z) * qs, bf16_lo(v[j].w) * qs, bf16_hi(v[j].w) * qs);
            }
            store_stream8(p.q + base + 512 * j, o);
        }
    }
}

template <bool NORM, int QMODE, bool E5M2>
bool launch_row_wave(const NormArgs& p, int rows, hipStream_t st) {
    const unsigned grid = ceil_div(rows, 4);
    switch (p.H / 512) {
#define CF_NORM_CASE(J) case J: k_norm_row_wave<J, NORM, QMODE, E5M2><<<grid, 256, 0, st>>>(p, rows); return true;
        CF_NORM_CASE(1) CF_NORM_CASE(2) CF_NORM_CASE(4) CF_NORM_CASE(8) CF_NORM_CASE(10) CF_NORM_CASE(14) CF_NORM_CASE(16)
#undef CF_NORM_CASE
        default: return false;
    }
}

template <bool NORM, int QMODE>
int launch_norm(const NormArgs& p, int rows, bool e5m2, hipStream_t st) {
    const int H = p.H;
    const int T = H < kNormMaxThreads ? H : kNormMaxThreads;
    bool vec = H % 8 == 0 && aligned16(p.x) && (!p.normed || aligned16(p.normed)) && (!NORM || aligned16(p.weight));
    if (QMODE != Q_NONE && (reinterpret_cast<uintptr_t>(p.q) & 7u) != 0) vec = false;
    if (vec && H % 512 == 0) {
        const bool done = e5m2 ? launch_row_wave<NORM, QMODE, true>(p, rows, st) : launch_row_wave<NORM, QMODE, false>(p, rows, st);
        if (done) return launch_status();
    }
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
