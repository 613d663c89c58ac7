// FP8 quantize family for gfx950: amax reduction, scale derivation, E4M3/E5M2
// quantize (plain, recording, per-row, per-1x128, per-128x128, fp32 input),
// delayed-scale history, clip probes, raw-byte E4M3 pack/unpack.
//
// All bulk kernels are HBM-bound: a lane moves 16 elements per step through
// two 128-bit loads and one 128-bit store, a wavefront reduces with xor
// shuffles, and a workgroup issues one atomic.
#include "common.hpp"
#include "internal.hpp"
#include <mutex>

namespace cf {
namespace {

constexpr int kThreads = 256;
constexpr int kVec = 16;            // elements per lane per step
constexpr unsigned kMaxBlocks = 4096;

__device__ __forceinline__ float block_max(float v, float* sh) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = sh[0];
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w) m = fmaxf(m, sh[w]);
        sh[0] = m;
    }
    __syncthreads();
    return sh[0];
}

// the same over per-wavefront integers (already reduced within each wavefront)
__device__ __forceinline__ int block_max_int(int wave_value, int* sh) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) sh[wave] = wave_value;
    __syncthreads();
    int m = sh[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) m = max(m, sh[w]);
    __syncthreads();
    return m;
}

struct Vec16 { uint4 lo, hi; };   // 16 bf16

__device__ __forceinline__ Vec16 load16(const uint16_t* p) {
    Vec16 v;
    v.lo = *reinterpret_cast<const uint4*>(p);
    v.hi = *reinterpret_cast<const uint4*>(p + 8);
    return v;
}
// the exact-erf GELU of 16 bf16 values, each result rounded to bf16 (what gelu_forward leaves in memory)
__device__ __forceinline__ Vec16 gelu16(const Vec16& v) {
    Vec16 g;
    g.lo = make_uint4(gelu2(v.lo.x), gelu2(v.lo.y), gelu2(v.lo.z), gelu2(v.lo.w));
    g.hi = make_uint4(gelu2(v.hi.x), gelu2(v.hi.y), gelu2(v.hi.z), gelu2(v.hi.w));
    return g;
}
__device__ __forceinline__ float amax16(const Vec16& v) {
    const uint32_t w[8] = {v.lo.x, v.lo.y, v.lo.z, v.lo.w, v.hi.x, v.hi.y, v.hi.z, v.hi.w};
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        m = fmaxf(m, fabsf(bf16_lo(w[i])));
        m = fmaxf(m, fabsf(bf16_hi(w[i])));
    }
    return m;
}
template <bool E5M2>
__device__ __forceinline__ uint4 quant16(const Vec16& v, float s) {
    const uint32_t w[8] = {v.lo.x, v.lo.y, v.lo.z, v.lo.w, v.hi.x, v.hi.y, v.hi.z, v.hi.w};
    uint4 o;
    o.x = cvt4_fp8<E5M2>(bf16_lo(w[0]) * s, bf16_hi(w[0]) * s, bf16_lo(w[1]) * s, bf16_hi(w[1]) * s);
    o.y = cvt4_fp8<E5M2>(bf16_lo(w[2]) * s, bf16_hi(w[2]) * s, bf16_lo(w[3]) * s, bf16_hi(w[3]) * s);
    o.z = cvt4_fp8<E5M2>(bf16_lo(w[4]) * s, bf16_hi(w[4]) * s, bf16_lo(w[5]) * s, bf16_hi(w[5]) * s);
    o.w = cvt4_fp8<E5M2>(bf16_lo(w[6]) * s, bf16_hi(w[6]) * s, bf16_lo(w[7]) * s, bf16_hi(w[7]) * s);
    return o;
}

__device__ __forceinline__ uint32_t absmax16(uint32_t acc, const Vec16& v) {
    acc = pk_absmax(pk_absmax(pk_absmax(pk_absmax(acc, v.lo.x), v.lo.y), v.lo.z), v.lo.w);
    return pk_absmax(pk_absmax(pk_absmax(pk_absmax(acc, v.hi.x), v.hi.y), v.hi.z), v.hi.w);
}
// quant16 for products known to hold no NaN
template <bool E5M2>
__device__ __forceinline__ uint4 quant16_finite(const Vec16& v, float s) {
    const uint32_t w[8] = {v.lo.x, v.lo.y, v.lo.z, v.lo.w, v.hi.x, v.hi.y, v.hi.z, v.hi.w};
    uint4 o;
    o.x = cvt4_fp8_finite<E5M2>(bf16_lo(w[0]) * s, bf16_hi(w[0]) * s, bf16_lo(w[1]) * s, bf16_hi(w[1]) * s);
    o.y = cvt4_fp8_finite<E5M2>(bf16_lo(w[2]) * s, bf16_hi(w[2]) * s, bf16_lo(w[3]) * s, bf16_hi(w[3]) * s);
    o.z = cvt4_fp8_finite<E5M2>(bf16_lo(w[4]) * s, bf16_hi(w[4]) * s, bf16_lo(w[5]) * s, bf16_hi(w[5]) * s);
    o.w = cvt4_fp8_finite<E5M2>(bf16_lo(w[6]) * s, bf16_hi(w[6]) * s, bf16_lo(w[7]) * s, bf16_hi(w[7]) * s);
    return o;
}

// Convert 16 elements with scale s, and (RECORD) fold their |max| into the running maxima: as bf16 bits when all
// 16 are finite (the common case: no per-element NaN handling at all), as a float maximum otherwise.
template <bool E5M2, bool RECORD>
__device__ __forceinline__ uint4 quant16_track(const Vec16& v, float s, bool scale_finite, int& max_bits, float& max_f) {
    const uint32_t acc = absmax16(0u, v);
    const int mb = static_cast<int>(max(acc & 0xffffu, acc >> 16));
    if (mb < 0x7f80 && scale_finite) {
        if constexpr (RECORD) max_bits = max(max_bits, mb);
        return quant16_finite<E5M2>(v, s);
    }
    if constexpr (RECORD) max_f = fmaxf(max_f, amax16(v));
    return quant16<E5M2>(v, s);
}

// ---- amax ------------------------------------------------------------------
// VEC: x is 16-byte aligned and the body is read as 16-element vectors; the
// n % 16 tail and the unaligned case go through the scalar loop.
// Launched with up to kAmaxThreads lanes per workgroup and one workgroup per CU: every workgroup ends in an
// atomic on the same address, and those serialise, so there should be few of them.
constexpr int kAmaxThreads = 1024;
constexpr unsigned kAmaxBlocks = 256;
template <bool VEC>
__global__ __launch_bounds__(kAmaxThreads) void k_amax_bf16(const uint16_t* __restrict__ x, size_t n,
                                                            float* __restrict__ amax) {
    __shared__ float sh[kAmaxThreads / 64];
    float local = 0.0f;
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t done = 0;
    if constexpr (VEC) {
        // four independent 32-byte loads per lane and step: few workgroups (few atomics) still keep HBM busy
        const size_t nvec = n / kVec;
        size_t i = tid;
        for (; i + 3 * stride < nvec; i += 4 * stride) {
            const Vec16 v0 = load16(x + i * kVec), v1 = load16(x + (i + stride) * kVec);
            const Vec16 v2 = load16(x + (i + 2 * stride) * kVec), v3 = load16(x + (i + 3 * stride) * kVec);
            local = fmaxf(fmaxf(local, fmaxf(amax16(v0), amax16(v1))), fmaxf(amax16(v2), amax16(v3)));
        }
        for (; i < nvec; i += stride) local = fmaxf(local, amax16(load16(x + i * kVec)));
        done = nvec * kVec;
    }
    for (size_t i = done + tid; i < n; i += stride) local = fmaxf(local, fabsf(bf16_to_f32(x[i])));
    const float m = block_max(local, sh);
    if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
}

__global__ __launch_bounds__(kThreads) void k_amax_f32(const float* __restrict__ x, size_t n,
                                                       float* __restrict__ amax, int vec) {
    __shared__ float sh[kThreads / 64];
    float local = 0.0f;
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t done = 0;
    if (vec) {
        const size_t nvec = n / 4;
        for (size_t i = tid; i < nvec; i += stride) {
            const float4 v = reinterpret_cast<const float4*>(x)[i];
            local = fmaxf(fmaxf(local, fabsf(v.x)), fmaxf(fmaxf(fabsf(v.y), fabsf(v.z)), fabsf(v.w)));
        }
        done = nvec * 4;
    }
    for (size_t i = done + tid; i < n; i += stride) local = fmaxf(local, fabsf(x[i]));
    const float m = block_max(local, sh);
    if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
}

__global__ void k_zero_f32(float* p) { *p = 0.0f; }

// ---- scalar-state kernels --------------------------------------------------
__global__ void k_scale_from_amax(const float* __restrict__ amax, float fp8_max,
                                  float* __restrict__ scale, float* __restrict__ descale) {
    const float a = fmaxf(*amax, 1e-12f);
    *scale = fp8_max / a;
    *descale = a / fp8_max;
}

// kernels/fp8.cu:105-142: ring append of max(amax, 1e-12), scale from the maximum of the entries filled so far
__device__ __forceinline__ void delayed_scale_update(float amax, float fp8_max, float* scale, float* descale,
                                                     float* history, int history_len, int* history_cursor,
                                                     int* history_count) {
    const float a = fmaxf(amax, 1e-12f);
    if (history_len <= 0) {
        *scale = fp8_max / a;
        *descale = a / fp8_max;
        return;
    }
    int cursor = *history_cursor;
    int count = *history_count;
    if (cursor < 0 || cursor >= history_len) cursor = 0;
    history[cursor] = a;
    cursor = (cursor + 1) % history_len;
    if (count < history_len) ++count;
    float hist_max = history[0];
    for (int i = 1; i < count; ++i) hist_max = fmaxf(hist_max, history[i]);
    hist_max = fmaxf(hist_max, 1e-12f);
    *history_cursor = cursor;
    *history_count = count;
    *scale = fp8_max / hist_max;
    *descale = hist_max / fp8_max;
}
__global__ void k_update_delayed_scale(const float* __restrict__ amax, float fp8_max,
                                       float* __restrict__ scale, float* __restrict__ descale,
                                       float* __restrict__ history, int history_len,
                                       int* __restrict__ history_cursor, int* __restrict__ history_count) {
    delayed_scale_update(*amax, fp8_max, scale, descale, history, history_len, history_cursor, history_count);
}

__global__ void k_clip_probe(const float* __restrict__ amax, const float* __restrict__ scale,
                             float fp8_max, float* __restrict__ stats) {
    const float a = *amax, s = *scale;
    stats[2] += 1.0f;
    if (fp8_max > 0.0f && s > 0.0f) {
        const float ratio = a * s / fp8_max;
        if (ratio > 1.0f) {
            stats[0] += 1.0f;
            if (ratio > stats[1]) stats[1] = ratio;
        }
    }
}

__global__ void k_calib_minmax(const float* __restrict__ amax, float* __restrict__ cmin,
                               float* __restrict__ cmax) {
    const float a = fmaxf(*amax, 1e-12f);
    *cmin = fminf(*cmin, a);
    *cmax = fmaxf(*cmax, a);
}

// ---- per-tensor quantize ---------------------------------------------------
template <bool E5M2, bool RECORD, bool VEC>
__global__ __launch_bounds__(kThreads) void k_quant(const uint16_t* __restrict__ x,
                                                    uint8_t* __restrict__ out,
                                                    const float* __restrict__ scale,
                                                    float* __restrict__ amax, size_t n) {
    __shared__ float sh[kThreads / 64];
    const float s = *scale;
    const bool s_finite = fabsf(s) < __uint_as_float(0x7f800000u);
    float local = 0.0f;
    int local_bits = 0;
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t done = 0;
    if constexpr (VEC) {
        const size_t nvec = n / kVec;
        for (size_t i = tid; i < nvec; i += stride) {
            const Vec16 v = load16(x + i * kVec);
            store_stream16(out + i * kVec, quant16_track<E5M2, RECORD>(v, s, s_finite, local_bits, local));
        }
        done = nvec * kVec;
    }
    for (size_t i = done + tid; i < n; i += stride) {
        const float v = bf16_to_f32(x[i]);
        if constexpr (RECORD) local = fmaxf(local, fabsf(v));
        out[i] = cvt1_fp8<E5M2>(v * s);
    }
    if constexpr (RECORD) {
        local = fmaxf(local, __uint_as_float(static_cast<uint32_t>(local_bits) << 16));
        const float m = block_max(local, sh);
        if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
    }
}

// The steady-state delayed-scaling step in one launch: quantize with the scale left by the previous call while
// recording this tensor's amax, then the workgroup that finishes last does what the reference spreads over
// separate launches and copies: snapshot the scale pair the quantize used, publish the amax, advance the history
// and the scale, and leave the running maximum and the arrival counter at zero for the next call.
struct DelayedStep {
    float* amax; float* scale; float* descale; float* scale_snapshot; float* descale_snapshot;
    float* history; int history_len; int* cursor; int* count;
    float* running_amax; unsigned* arrived;     // both zero between calls
    float fp8_max;
};
// Every workgroup ends in an atomic on the arrival counter, and atomics on one address serialise: one large
// workgroup per CU (as for the amax kernel) keeps that tail to a few microseconds.
template <bool E5M2, bool VEC>
__global__ __launch_bounds__(kAmaxThreads) void k_quant_delayed_step(const uint16_t* __restrict__ x, uint8_t* __restrict__ out,
                                                                     size_t n, const DelayedStep d) {
    __shared__ float sh[kAmaxThreads / 64];
    const float s = *d.scale;
    const bool s_finite = fabsf(s) < __uint_as_float(0x7f800000u);
    // What the workgroup that arrives last needs of the slot's state is read now, by every workgroup's first lane, so
    // that no chain of dependent loads is left for the end: the state only changes in that last step, i.e. between
    // launches.  pre_max = the history maximum over the entries the update will look at, without the one it overwrites.
    float pre_descale = 0.0f, pre_max = 0.0f;
    int pre_cursor = 0, pre_count = 0;
    if (threadIdx.x == 0) {
        pre_descale = *d.descale;
        if (d.history_len > 0) {
            pre_cursor = *d.cursor;
            pre_count = *d.count;
            if (pre_cursor < 0 || pre_cursor >= d.history_len) pre_cursor = 0;
            if (pre_count < d.history_len) ++pre_count;
            for (int i = 0; i < pre_count; ++i)
                if (i != pre_cursor) pre_max = fmaxf(pre_max, d.history[i]);
        }
    }
    float local = 0.0f;
    int local_bits = 0;
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t done = 0;
    if constexpr (VEC) {
        const size_t nvec = n / kVec;
        for (size_t i = tid; i < nvec; i += stride) {
            const Vec16 v = load16(x + i * kVec);
            store_stream16(out + i * kVec, quant16_track<E5M2, true>(v, s, s_finite, local_bits, local));
        }
        done = nvec * kVec;
    }
    for (size_t i = done + tid; i < n; i += stride) {
        const float v = bf16_to_f32(x[i]);
        local = fmaxf(local, fabsf(v));
        out[i] = cvt1_fp8<E5M2>(v * s);
    }
    local = fmaxf(local, __uint_as_float(static_cast<uint32_t>(local_bits) << 16));
    const float m = block_max(local, sh);
    if (threadIdx.x == 0) {
        if (arrive_with_max(d.running_amax, d.arrived, m, gridDim.x)) {
            const float amax = atomic_load_agent(d.running_amax);
            *d.scale_snapshot = s;                           // every workgroup read the same pair at its start
            *d.descale_snapshot = pre_descale;
            *d.amax = amax;
            // delayed_scale_update() on the state read at the start
            const float a = fmaxf(amax, 1e-12f);
            float hist_max = a;
            if (d.history_len > 0) {
                d.history[pre_cursor] = a;
                hist_max = fmaxf(pre_cursor < pre_count ? fmaxf(pre_max, a) : pre_max, 1e-12f);
                *d.cursor = (pre_cursor + 1) % d.history_len;
                *d.count = pre_count;
            }
            *d.scale = d.fp8_max / hist_max;
            *d.descale = hist_max / d.fp8_max;
            *d.running_amax = 0.0f;
            *d.arrived = 0u;
        }
    }
}

// The same step for a bank of experts in one launch: the rows of expert e (counts[e] of them, from row offsets[e] of a
// compact [total_rows, K] buffer) are one tensor with its own delayed-scaling state block (the word layout of
// cf_act_slot's device block; block e starts e * stride words after the first).  blockIdx.y = expert, gridDim.x
// workgroups share an expert's rows; an expert without rows is left alone, state included (the reference's loop skips
// it before fp8_quant_act, src/trainer.cu:6887-6888).  GELU: the tensor quantized is bf16(gelu(x)) (gelu_forward in
// place, then fp8_quant_act, :6910-6918).  RECOMPUTE: the backward's second pass, with the snapshot scale and no side
// effects (:4736-4743).  row_descale[r] = the descale the GEMM that consumes row r dequantizes with (the expert's
// descale_snapshot, :6921-6924).
template <bool E5M2, bool GELU, bool RECOMPUTE>
__global__ __launch_bounds__(kThreads) void k_grouped_quant_delayed(const uint16_t* __restrict__ x, uint8_t* __restrict__ out, int K,
                                                                    const int* __restrict__ counts, const int* __restrict__ offsets,
                                                                    int total_rows, float* __restrict__ states, int stride,
                                                                    int history_len, float fp8_max, float* __restrict__ row_descale) {
    __shared__ float sh[kThreads / 64];
    const int e = blockIdx.y;
    const int first = offsets[e];
    const int rows = first >= 0 && first < total_rows ? min(counts[e], total_rows - first) : 0;
    if (rows <= 0) return;
    float* st = states + static_cast<size_t>(e) * stride;
    const float s = st[RECOMPUTE ? slotw::SCALE_SNAP : slotw::SCALE];
    const float ds = st[RECOMPUTE ? slotw::DESCALE_SNAP : slotw::DESCALE];
    const bool s_finite = fabsf(s) < __uint_as_float(0x7f800000u);
    float pre_max = 0.0f;
    int pre_cursor = 0, pre_count = 0;
    if (!RECOMPUTE && threadIdx.x == 0 && history_len > 0) {
        pre_cursor = reinterpret_cast<const int*>(st)[slotw::CURSOR];
        pre_count = reinterpret_cast<const int*>(st)[slotw::COUNT];
        if (pre_cursor < 0 || pre_cursor >= history_len) pre_cursor = 0;
        if (pre_count < history_len) ++pre_count;
        for (int i = 0; i < pre_count; ++i)
            if (i != pre_cursor) pre_max = fmaxf(pre_max, st[slotw::HISTORY + i]);
    }
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t stride_t = static_cast<size_t>(gridDim.x) * kThreads;
    for (size_t r = tid; r < static_cast<size_t>(rows); r += stride_t) row_descale[first + r] = ds;
    const uint16_t* xe = x + static_cast<size_t>(first) * K;
    uint8_t* oe = out + static_cast<size_t>(first) * K;
    const size_t nvec = static_cast<size_t>(rows) * K / kVec;       // K % 16 == 0
    float local = 0.0f;
    int local_bits = 0;
    for (size_t i = tid; i < nvec; i += stride_t) {
        Vec16 v = load16(xe + i * kVec);
        if constexpr (GELU) v = gelu16(v);
        store_stream16(oe + i * kVec, quant16_track<E5M2, !RECOMPUTE>(v, s, s_finite, local_bits, local));
    }
    if constexpr (!RECOMPUTE) {
        local = fmaxf(local, __uint_as_float(static_cast<uint32_t>(local_bits) << 16));
        const float m = block_max(local, sh);
        if (threadIdx.x == 0) {
            unsigned* arrived = reinterpret_cast<unsigned*>(st) + slotw::ARRIVED;
            if (arrive_with_max(st + slotw::RUNNING, arrived, m, gridDim.x)) {
                const float amax = atomic_load_agent(st + slotw::RUNNING);
                st[slotw::SCALE_SNAP] = s;
                st[slotw::DESCALE_SNAP] = ds;
                st[slotw::AMAX] = amax;
                const float a = fmaxf(amax, 1e-12f);
                float hist_max = a;
                if (history_len > 0) {
                    st[slotw::HISTORY + pre_cursor] = a;
                    hist_max = fmaxf(pre_cursor < pre_count ? fmaxf(pre_max, a) : pre_max, 1e-12f);
                    reinterpret_cast<int*>(st)[slotw::CURSOR] = (pre_cursor + 1) % history_len;
                    reinterpret_cast<int*>(st)[slotw::COUNT] = pre_count;
                }
                st[slotw::SCALE] = fp8_max / hist_max;
                st[slotw::DESCALE] = hist_max / fp8_max;
                st[slotw::RUNNING] = 0.0f;
                *arrived = 0u;
            }
        }
    }
}

template <bool E5M2>
__global__ __launch_bounds__(kThreads) void k_quant_f32(const float* __restrict__ x,
                                                        uint8_t* __restrict__ out,
                                                        const float* __restrict__ scale, size_t n,
                                                        int vec) {
    const float s = *scale;
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t done = 0;
    if (vec) {
        const size_t nvec = n / 4;
        for (size_t i = tid; i < nvec; i += stride) {
            const float4 v = reinterpret_cast<const float4*>(x)[i];
            __builtin_nontemporal_store(cvt4_fp8<E5M2>(v.x * s, v.y * s, v.z * s, v.w * s), reinterpret_cast<uint32_t*>(out) + i);
        }
        done = nvec * 4;
    }
    for (size_t i = done + tid; i < n; i += stride) out[i] = cvt1_fp8<E5M2>(x[i] * s);
}

__global__ __launch_bounds__(kThreads) void k_elem_clip_count(const uint16_t* __restrict__ x,
                                                              const float* __restrict__ scale,
                                                              float fp8_max, size_t n,
                                                              float* __restrict__ out) {
    const float s = *scale;
    int clipped = 0;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        if (fabsf(bf16_to_f32(x[i])) * s > fp8_max) ++clipped;
    clipped = wave_sum_i(clipped);
    if ((threadIdx.x & 63) == 0 && clipped) atomicAdd(&out[0], static_cast<float>(clipped));
    if (blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&out[1], static_cast<float>(n));
}

// ---- per-row quantize ---------------------------------------------------------
// One wavefront per row.  The row stays in registers between the amax pass and
// the convert pass, so HBM sees 2 B read + 1 B written per element.
// MAXS = register-resident steps of 64 lanes x 16 elements.
// GELU: the row quantized is bf16(gelu(x)), computed on the way in (the activation between an expert's two
// projections is never written as bf16).
template <bool E5M2, int MAXS, bool GELU = false>
__global__ __launch_bounds__(kThreads) void k_quant_rows(const uint16_t* __restrict__ x, int rows, int K,
                                                         uint8_t* __restrict__ out,
                                                         float* __restrict__ scale,
                                                         float* __restrict__ descale) {
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const uint16_t* xr = x + static_cast<size_t>(row) * K;
    uint8_t* outr = out + static_cast<size_t>(row) * K;
    Vec16 v[MAXS];
    uint32_t acc = 0;                 // packed integer maximum of |bf16|: one instruction per pair
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = (s * 64 + lane) * kVec;
        if (k < K) {
            v[s] = load16(xr + k);
            if constexpr (GELU) v[s] = gelu16(v[s]);
            acc = absmax16(acc, v[s]);
        }
    }
    const int mbits = wave_absmax_bits(acc);
    const bool finite = mbits < 0x7f80;
    float m = __uint_as_float(static_cast<uint32_t>(mbits) << 16);
    if (!finite) {                    // a float maximum ignores NaNs
        float local = 0.0f;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
            if ((s * 64 + lane) * kVec < K) local = fmaxf(local, amax16(v[s]));
        m = wave_max(local);
    }
    constexpr float fmax_ = E5M2 ? 57344.0f : 448.0f;
    const float a = fmaxf(m, 1e-12f);
    const float sc = fmax_ / a;
    if (lane == 0) { scale[row] = sc; descale[row] = a / fmax_; }
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = (s * 64 + lane) * kVec;
        if (k < K) store_stream16(outr + k, finite ? quant16_finite<E5M2>(v[s], sc) : quant16<E5M2>(v[s], sc));
    }
}

// GELU + per-row quantize for many rows: the exact-erf GELU of a bf16 value is a function of its 16 bits, so a
// workgroup that stays on its CU builds the table of all 65536 results once (128 KiB of LDS, 64 erff per lane) and then
// looks every element up instead of evaluating erff, which is what the plain form above waits for (about 40 vector
// instructions per element).  Same bits: the table holds bf16(gelu_fwd(x)) for every x.
constexpr int kLutThreads = 1024;
__global__ __launch_bounds__(kLutThreads) void k_gelu_quant_rows_lut(const uint16_t* __restrict__ x, int rows, int K,
                                                                     uint8_t* __restrict__ out, float* __restrict__ scale,
                                                                     float* __restrict__ descale) {
    extern __shared__ uint16_t lut[];
    for (int i = threadIdx.x; i < 65536; i += kLutThreads) lut[i] = f32_to_bf16(gelu_fwd(bf16_to_f32(static_cast<uint16_t>(i))));
    __syncthreads();
    auto look2 = [&](uint32_t pair) { return static_cast<uint32_t>(lut[pair & 0xffffu]) | (static_cast<uint32_t>(lut[pair >> 16]) << 16); };
    constexpr int MAXS = 4;
    const int lane = threadIdx.x & 63;
    const int waves = gridDim.x * (kLutThreads / 64);
    for (int row = blockIdx.x * (kLutThreads / 64) + (threadIdx.x >> 6); row < rows; row += waves) {
        const uint16_t* xr = x + static_cast<size_t>(row) * K;
        uint8_t* outr = out + static_cast<size_t>(row) * K;
        Vec16 v[MAXS];
        uint32_t acc = 0;
#pragma unroll
        for (int s = 0; s < MAXS; ++s) {
            const int k = (s * 64 + lane) * kVec;
            if (k < K) v[s] = load16(xr + k);
        }
#pragma unroll
        for (int s = 0; s < MAXS; ++s) {
            const int k = (s * 64 + lane) * kVec;
            if (k < K) {
                v[s].lo = make_uint4(look2(v[s].lo.x), look2(v[s].lo.y), look2(v[s].lo.z), look2(v[s].lo.w));
                v[s].hi = make_uint4(look2(v[s].hi.x), look2(v[s].hi.y), look2(v[s].hi.z), look2(v[s].hi.w));
                acc = absmax16(acc, v[s]);
            }
        }
        const int mbits = wave_absmax_bits(acc);
        const bool finite = mbits < 0x7f80;
        float m = __uint_as_float(static_cast<uint32_t>(mbits) << 16);
        if (!finite) {                    // a float maximum ignores NaNs
            float local = 0.0f;
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
                if ((s * 64 + lane) * kVec < K) local = fmaxf(local, amax16(v[s]));
            m = wave_max(local);
        }
        const float a = fmaxf(m, 1e-12f);
        const float sc = 448.0f / a;
        if (lane == 0) { scale[row] = sc; descale[row] = a / 448.0f; }
#pragma unroll
        for (int s = 0; s < MAXS; ++s) {
            const int k = (s * 64 + lane) * kVec;
            if (k < K) store_stream16(outr + k, finite ? quant16_finite<false>(v[s], sc) : quant16<false>(v[s], sc));
        }
    }
}

// k_grouped_quant_delayed with GELU for large banks, on the same table: one workgroup per CU stays resident, builds
// the 65536-entry table once and then takes the (expert, part) items w = blockIdx.x, blockIdx.x + gridDim.x, ...
// (part p of `per` covers the expert's 16-element vectors p * 1024 + lane, stepping per * 1024).  An item ends as a
// workgroup of the plain form does: maximum into the slot's running amax, one arrival; the item that arrives last of an
// expert's `per` updates the slot.  The slot's state changes only in that last step, and only after every item of the
// expert has arrived, so what a workgroup reads of it at the start of the kernel (row range and scale pair of every
// expert, into LDS, under the table build) is the state the call started with; the history is read by the last
// arrival alone.  Same bits as the plain form: the table holds bf16(gelu_fwd(x)) for every x.
constexpr int kLutMaxExperts = 1024;
template <bool E5M2, bool RECOMPUTE>
__global__ __launch_bounds__(kLutThreads) void k_grouped_gelu_quant_delayed_lut(const uint16_t* __restrict__ x, uint8_t* __restrict__ out,
                                                                               int K, const int* __restrict__ counts,
                                                                               const int* __restrict__ offsets, int total_rows,
                                                                               int num_experts, int per, float* __restrict__ states,
                                                                               int stride, int history_len, float fp8_max,
                                                                               float* __restrict__ row_descale) {
    extern __shared__ uint16_t lut[];
    __shared__ float sh[2][kLutThreads / 64];
    __shared__ int sh_first[kLutMaxExperts], sh_rows[kLutMaxExperts];
    __shared__ float sh_scale[kLutMaxExperts], sh_descale[kLutMaxExperts];
    for (int e = threadIdx.x; e < num_experts; e += kLutThreads) {
        const int first = offsets[e];
        sh_first[e] = first;
        sh_rows[e] = first >= 0 && first < total_rows ? min(counts[e], total_rows - first) : 0;
        const float* st = states + static_cast<size_t>(e) * stride;
        sh_scale[e] = st[RECOMPUTE ? slotw::SCALE_SNAP : slotw::SCALE];
        sh_descale[e] = st[RECOMPUTE ? slotw::DESCALE_SNAP : slotw::DESCALE];
    }
    for (int i = threadIdx.x; i < 65536; i += kLutThreads) lut[i] = f32_to_bf16(gelu_fwd(bf16_to_f32(static_cast<uint16_t>(i))));
    __syncthreads();
    auto look2 = [&](uint32_t pair) { return static_cast<uint32_t>(lut[pair & 0xffffu]) | (static_cast<uint32_t>(lut[pair >> 16]) << 16); };
    const int items = num_experts * per;
    int parity = 0;
    for (int w = blockIdx.x; w < items; w += gridDim.x) {
        const int e = w / per, part = w - e * per;
        const int rows = sh_rows[e];
        if (rows <= 0) continue;                                     // uniform over the workgroup
        const int first = sh_first[e];
        const float s = sh_scale[e], ds = sh_descale[e];
        const bool s_finite = fabsf(s) < __uint_as_float(0x7f800000u);
        const size_t tid = static_cast<size_t>(part) * kLutThreads + threadIdx.x;
        const size_t stride_t = static_cast<size_t>(per) * kLutThreads;
        for (size_t r = tid; r < static_cast<size_t>(rows); r += stride_t) row_descale[first + r] = ds;
        const uint16_t* xe = x + static_cast<size_t>(first) * K;
        uint8_t* oe = out + static_cast<size_t>(first) * K;
        const size_t nvec = static_cast<size_t>(rows) * K / kVec;       // K % 16 == 0
        float local = 0.0f;
        int local_bits = 0;
        constexpr int kBatch = 4;                                    // loads in flight per lane
        for (size_t i0 = tid; i0 < nvec; i0 += kBatch * stride_t) {
            Vec16 v[kBatch];
#pragma unroll
            for (int b = 0; b < kBatch; ++b)
                if (i0 + b * stride_t < nvec) v[b] = load16(xe + (i0 + b * stride_t) * kVec);
#pragma unroll
            for (int b = 0; b < kBatch; ++b) {
                const size_t i = i0 + b * stride_t;
                if (i < nvec) {
                    v[b].lo = make_uint4(look2(v[b].lo.x), look2(v[b].lo.y), look2(v[b].lo.z), look2(v[b].lo.w));
                    v[b].hi = make_uint4(look2(v[b].hi.x), look2(v[b].hi.y), look2(v[b].hi.z), look2(v[b].hi.w));
                    store_stream16(oe + i * kVec, quant16_track<E5M2, !RECOMPUTE>(v[b], s, s_finite, local_bits, local));
                }
            }
        }
        if constexpr (!RECOMPUTE) {
            local = fmaxf(local, __uint_as_float(static_cast<uint32_t>(local_bits) << 16));
            // the two halves of sh alternate between items: the other wavefronts go on to the next item while the
            // first lane is busy with the arrival
            const float m = block_max(local, sh[parity]);
            parity ^= 1;
            if (threadIdx.x == 0) {
                float* st = states + static_cast<size_t>(e) * stride;
                unsigned* arrived = reinterpret_cast<unsigned*>(st) + slotw::ARRIVED;
                if (arrive_with_max(st + slotw::RUNNING, arrived, m, static_cast<unsigned>(per))) {
                    const float amax = atomic_load_agent(st + slotw::RUNNING);
                    st[slotw::SCALE_SNAP] = s;
                    st[slotw::DESCALE_SNAP] = ds;
                    st[slotw::AMAX] = amax;
                    const float a = fmaxf(amax, 1e-12f);
                    float hist_max = a;
                    if (history_len > 0) {
                        int cursor = reinterpret_cast<const int*>(st)[slotw::CURSOR];
                        int count = reinterpret_cast<const int*>(st)[slotw::COUNT];
                        if (cursor < 0 || cursor >= history_len) cursor = 0;
                        if (count < history_len) ++count;
                        float pre_max = 0.0f;
                        for (int i = 0; i < count; ++i)
                            if (i != cursor) pre_max = fmaxf(pre_max, st[slotw::HISTORY + i]);
                        st[slotw::HISTORY + cursor] = a;
                        hist_max = fmaxf(cursor < count ? fmaxf(pre_max, a) : pre_max, 1e-12f);
                        reinterpret_cast<int*>(st)[slotw::CURSOR] = (cursor + 1) % history_len;
                        reinterpret_cast<int*>(st)[slotw::COUNT] = count;
                    }
                    st[slotw::SCALE] = fp8_max / hist_max;
                    st[slotw::DESCALE] = hist_max / fp8_max;
                    st[slotw::RUNNING] = 0.0f;
                    *arrived = 0u;
                }
            }
        }
    }
}

// Long rows (4096 < K <= 32768): one workgroup of four wavefronts per row, the row still register-resident (four or
// eight steps per lane instead of sixteen or more, so more wavefronts fit a SIMD); the row maximum crosses the
// wavefronts through LDS.
template <bool E5M2, int MAXS, bool GELU = false>      // MAXS steps of 256 lanes x 16 elements: 4 covers K <= 16384, 8 covers K <= 32768
__global__ __launch_bounds__(kThreads) void k_quant_rows_block(const uint16_t* __restrict__ x, int K,
                                                               uint8_t* __restrict__ out,
                                                               float* __restrict__ scale,
                                                               float* __restrict__ descale) {
    __shared__ int sh_bits[kThreads / 64];
    __shared__ float sh_max[kThreads / 64];
    const int row = blockIdx.x, tid = threadIdx.x;
    const uint16_t* xr = x + static_cast<size_t>(row) * K;
    uint8_t* outr = out + static_cast<size_t>(row) * K;
    Vec16 v[MAXS];
    uint32_t acc = 0;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = (s * kThreads + tid) * kVec;
        if (k < K) {
            v[s] = load16(xr + k);
            if constexpr (GELU) v[s] = gelu16(v[s]);
            acc = absmax16(acc, v[s]);
        }
    }
    const int wbits = wave_absmax_bits(acc);
    if ((tid & 63) == 0) sh_bits[tid >> 6] = wbits;
    __syncthreads();
    const int mbits = max(max(sh_bits[0], sh_bits[1]), max(sh_bits[2], sh_bits[3]));
    const bool finite = mbits < 0x7f80;
    float m = __uint_as_float(static_cast<uint32_t>(mbits) << 16);
    if (!finite) {                    // a float maximum ignores NaNs
        float local = 0.0f;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
            if ((s * kThreads + tid) * kVec < K) local = fmaxf(local, amax16(v[s]));
        local = wave_max(local);
        if ((tid & 63) == 0) sh_max[tid >> 6] = local;
        __syncthreads();
        m = fmaxf(fmaxf(sh_max[0], sh_max[1]), fmaxf(sh_max[2], sh_max[3]));
    }
    constexpr float fmax_ = E5M2 ? 57344.0f : 448.0f;
    const float a = fmaxf(m, 1e-12f);
    const float sc = fmax_ / a;
    if (tid == 0) { scale[row] = sc; descale[row] = a / fmax_; }
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = (s * kThreads + tid) * kVec;
        if (k < K) store_stream16(outr + k, finite ? quant16_finite<E5M2>(v[s], sc) : quant16<E5M2>(v[s], sc));
    }
}

// Any K, any alignment: one workgroup per row, two passes over the row.
template <bool E5M2, bool GELU = false>
__global__ __launch_bounds__(kThreads) void k_quant_rows_generic(const uint16_t* __restrict__ x, int K,
                                                                 uint8_t* __restrict__ out,
                                                                 float* __restrict__ scale,
                                                                 float* __restrict__ descale) {
    __shared__ float sh[kThreads / 64];
    const int row = blockIdx.x;
    const uint16_t* xr = x + static_cast<size_t>(row) * K;
    uint8_t* outr = out + static_cast<size_t>(row) * K;
    auto value = [&](int k) {
        const float v = bf16_to_f32(xr[k]);
        return GELU ? bf16_to_f32(f32_to_bf16(gelu_fwd(v))) : v;
    };
    float local = 0.0f;
    for (int k = threadIdx.x; k < K; k += blockDim.x) local = fmaxf(local, fabsf(value(k)));
    constexpr float fmax_ = E5M2 ? 57344.0f : 448.0f;
    const float a = fmaxf(block_max(local, sh), 1e-12f);
    const float sc = fmax_ / a;
    if (threadIdx.x == 0) { scale[row] = sc; descale[row] = a / fmax_; }
    for (int k = threadIdx.x; k < K; k += blockDim.x) outr[k] = cvt1_fp8<E5M2>(value(k) * sc);
}

// ---- 1x128 groups ------------------------------------------------------------
// K % 128 == 0, 16-byte aligned rows: a group is 8 neighbouring lanes.
__global__ __launch_bounds__(kThreads) void k_quant_1x128(const uint16_t* __restrict__ x, size_t ngroups,
                                                          uint8_t* __restrict__ out,
                                                          float* __restrict__ scale,
                                                          float* __restrict__ descale) {
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    const size_t nvec = ngroups * 8;
    // every lane of a wave runs the same number of iterations (nvec % 8 == 0, stride % 64 == 0)
    for (size_t i = tid; i < ((nvec + 63) / 64) * 64; i += stride) {
        const bool live = i < nvec;
        Vec16 v = {};
        if (live) v = load16(x + i * kVec);
        // group maximum as bf16 bits (packed integer maximum of the sign-cleared pairs); a group with a NaN or
        // an infinity (bits >= 0x7f80) takes the float maximum, which ignores NaNs, and the NaN-restoring convert
        const uint32_t acc = absmax16(0u, v);
        int mb = static_cast<int>(max(acc & 0xffffu, acc >> 16));
        mb = max(mb, __shfl_xor(mb, 1, kWave));
        mb = max(mb, __shfl_xor(mb, 2, kWave));
        mb = max(mb, __shfl_xor(mb, 4, kWave));
        const bool finite = mb < 0x7f80;
        float m = __uint_as_float(static_cast<uint32_t>(mb) << 16);
        if (!finite) {
            m = amax16(v);
            m = fmaxf(m, __shfl_xor(m, 1, kWave));
            m = fmaxf(m, __shfl_xor(m, 2, kWave));
            m = fmaxf(m, __shfl_xor(m, 4, kWave));
        }
        const float a = fmaxf(m, 1e-12f);
        const float sc = 448.0f / a;
        if (live) {
            if ((i & 7) == 0) { scale[i >> 3] = sc; descale[i >> 3] = a / 448.0f; }
            store_stream16(out + i * kVec, finite ? quant16_finite<false>(v, sc) : quant16<false>(v, sc));
        }
    }
}

// ragged K or unaligned rows: one wavefront per group
__global__ __launch_bounds__(kThreads) void k_quant_1x128_generic(const uint16_t* __restrict__ x, int rows,
                                                                  int K, uint8_t* __restrict__ out,
                                                                  float* __restrict__ scale,
                                                                  float* __restrict__ descale) {
    const int kb = (K + 127) / 128;
    const size_t g = static_cast<size_t>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
    if (g >= static_cast<size_t>(rows) * kb) return;
    const int lane = threadIdx.x & 63;
    const int r = static_cast<int>(g / kb), b = static_cast<int>(g % kb);
    const size_t base = static_cast<size_t>(r) * K + static_cast<size_t>(b) * 128;
    const int len = min(128, K - b * 128);
    float v0 = lane < len ? bf16_to_f32(x[base + lane]) : 0.0f;
    float v1 = lane + 64 < len ? bf16_to_f32(x[base + lane + 64]) : 0.0f;
    const float a = fmaxf(wave_max(fmaxf(fabsf(v0), fabsf(v1))), 1e-12f);
    const float sc = 448.0f / a;
    if (lane == 0) { scale[g] = sc; descale[g] = a / 448.0f; }
    if (lane < len) out[base + lane] = cvt1_fp8<false>(v0 * sc);
    if (lane + 64 < len) out[base + lane + 64] = cvt1_fp8<false>(v1 * sc);
}

// ---- 128x128 blocks ------------------------------------------------------------
// One workgroup per block; a thread holds a 4 x 16 slice in registers.
__global__ __launch_bounds__(kThreads) void k_quant_128x128(const uint16_t* __restrict__ x, int rows, int K,
                                                            uint8_t* __restrict__ out,
                                                            float* __restrict__ scale,
                                                            float* __restrict__ descale, int vec) {
    __shared__ float sh[kThreads / 64];
    const int kb = (K + 127) / 128;
    const int br = blockIdx.x / kb, bk = blockIdx.x % kb;
    const int r0 = br * 128, k0 = bk * 128;
    const int tr = threadIdx.x >> 3, tc = (threadIdx.x & 7) * kVec;    // 32 rows x 8 lanes per pass
    float local = 0.0f;
    if (vec) {
        Vec16 v[4];
        uint32_t acc = 0;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int r = r0 + p * 32 + tr;
            v[p] = Vec16{};
            if (r < rows) v[p] = load16(x + static_cast<size_t>(r) * K + k0 + tc);
            acc = absmax16(acc, v[p]);
        }
        // block maximum as bf16 bits; blocks holding a NaN or an infinity redo it as a float maximum (NaNs ignored)
        const int mb = block_max_int(wave_absmax_bits(acc), reinterpret_cast<int*>(sh));
        const bool finite = mb < 0x7f80;
        float m = __uint_as_float(static_cast<uint32_t>(mb) << 16);
        if (!finite) {
#pragma unroll
            for (int p = 0; p < 4; ++p) local = fmaxf(local, amax16(v[p]));
            m = block_max(local, sh);
        }
        const float a = fmaxf(m, 1e-12f);
        const float sc = 448.0f / a;
        if (threadIdx.x == 0) { scale[blockIdx.x] = sc; descale[blockIdx.x] = a / 448.0f; }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int r = r0 + p * 32 + tr;
            if (r < rows)
                store_stream16(out + static_cast<size_t>(r) * K + k0 + tc, finite ? quant16_finite<false>(v[p], sc) : quant16<false>(v[p], sc));
        }
    } else {
        const int klen = min(128, K - k0), rlen = min(128, rows - r0);
        for (int i = threadIdx.x; i < rlen * 128; i += blockDim.x) {
            const int r = i >> 7, k = i & 127;
            if (k < klen) local = fmaxf(local, fabsf(bf16_to_f32(x[static_cast<size_t>(r0 + r) * K + k0 + k])));
        }
        const float a = fmaxf(block_max(local, sh), 1e-12f);
        const float sc = 448.0f / a;
        if (threadIdx.x == 0) { scale[blockIdx.x] = sc; descale[blockIdx.x] = a / 448.0f; }
        for (int i = threadIdx.x; i < rlen * 128; i += blockDim.x) {
            const int r = i >> 7, k = i & 127;
            if (k < klen) {
                const size_t idx = static_cast<size_t>(r0 + r) * K + k0 + k;
                out[idx] = cvt1_fp8<false>(bf16_to_f32(x[idx]) * sc);
            }
        }
    }
}

// ---- raw-byte E4M3 storage path --------------------------------------------------
// The byte contract pack(): like the saturating convert for finite input,
// nonfinite input -> sign|0x7f and flagged.
__device__ __forceinline__ uint8_t pack_raw(float v, bool& finite) {
    const uint32_t bits = __float_as_uint(v);
    finite = (bits & 0x7f800000u) != 0x7f800000u;
    if (!finite) return static_cast<uint8_t>(((bits >> 24) & 0x80u) | 0x7fu);
    return cvt1_fp8<false>(v);
}

__global__ __launch_bounds__(kThreads) void k_raw_stats(const uint16_t* __restrict__ x, size_t n,
                                                        float* __restrict__ amax, int* __restrict__ bad) {
    __shared__ float sh[kThreads / 64];
    float local = 0.0f;
    int nbad = 0;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const float v = bf16_to_f32(x[i]);
        if ((__float_as_uint(v) & 0x7f800000u) == 0x7f800000u) ++nbad;
        else local = fmaxf(local, fabsf(v));
    }
    nbad = wave_sum_i(nbad);
    if ((threadIdx.x & 63) == 0 && nbad) atomicAdd(bad, nbad);
    const float m = block_max(local, sh);
    if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
}

template <bool DEQUANT>
__global__ __launch_bounds__(kThreads) void k_raw_pack(const uint16_t* __restrict__ x,
                                                       uint8_t* __restrict__ out,
                                                       uint16_t* __restrict__ dequant,
                                                       const float* __restrict__ scale,
                                                       const float* __restrict__ descale,
                                                       int* __restrict__ bad, size_t n) {
    const float s = *scale;
    const float d = DEQUANT ? *descale : 0.0f;
    int nbad = 0;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        bool fin;
        const uint8_t code = pack_raw(bf16_to_f32(x[i]) * s, fin);
        out[i] = code;
        if constexpr (DEQUANT) dequant[i] = f32_to_bf16(e4m3_to_f32(code) * d);
        if (!fin) ++nbad;
    }
    nbad = wave_sum_i(nbad);
    if ((threadIdx.x & 63) == 0 && nbad) atomicAdd(bad, nbad);
}

__global__ __launch_bounds__(kThreads) void k_raw_unpack(const uint8_t* __restrict__ in,
                                                         const float* __restrict__ descale,
                                                         uint16_t* __restrict__ out, size_t n) {
    const float d = *descale;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        out[i] = f32_to_bf16(e4m3_to_f32(in[i]) * d);
}

__global__ void k_zero_raw(float* amax, int* bad) { *amax = 0.0f; *bad = 0; }

unsigned blocks_for(size_t items) {
    const size_t b = (items + kThreads - 1) / kThreads;
    return static_cast<unsigned>(b < 1 ? 1 : (b > kMaxBlocks ? kMaxBlocks : b));
}

template <bool E5M2, bool RECORD>
int launch_quant(const uint16_t* x, void* out, const float* scale, float* amax, size_t n, cf_stream_t st) {
    if (n == 0) return CF_OK;
    if (!x || !out || !scale || (RECORD && !amax)) return CF_ERR_INVALID_ARG;
    auto* o = static_cast<uint8_t*>(out);
    if (aligned16(x) && aligned16(out))
        k_quant<E5M2, RECORD, true><<<blocks_for((n + kVec - 1) / kVec), kThreads, 0, as_stream(st)>>>(x, o, scale, amax, n);
    else
        k_quant<E5M2, RECORD, false><<<blocks_for(n), kThreads, 0, as_stream(st)>>>(x, o, scale, amax, n);
    return launch_status();
}

// per-row quantize: the register-resident forms where the row fits, the two-pass form otherwise
template <bool E5M2, bool GELU>
int launch_quant_rows(const uint16_t* d_x, int rows, int K, void* d_out, float* d_scale, float* d_descale, cf_stream_t stream) {
    if (rows < 0 || K < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0) return CF_OK;
    if (!d_scale || !d_descale || (K > 0 && (!d_x || !d_out))) return CF_ERR_INVALID_ARG;
    auto* o = static_cast<uint8_t*>(d_out);
    hipStream_t st = as_stream(stream);
    const bool vec = aligned16(d_x) && aligned16(d_out) && K % kVec == 0 && K > 0;
    const unsigned grid = ceil_div(rows, kThreads / 64);
    if constexpr (GELU && !E5M2) {
        // enough rows to pay for 256 tables of 65536 entries (each costs what 64 rows of 1024 elements cost directly)
        if (vec && K <= 4 * 1024 && static_cast<size_t>(rows) * K >= (64u << 20)) {
            static std::once_flag once;
            static hipError_t err = hipSuccess;
            static int cus = 256;
            std::call_once(once, [] {
                err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gelu_quant_rows_lut),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
                int dev = 0, n = 0;
                if (hipGetDevice(&dev) == hipSuccess &&
                    hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
                    cus = n;
            });
            if (err != hipSuccess) return static_cast<int>(err);
            k_gelu_quant_rows_lut<<<cus, kLutThreads, 128 * 1024, st>>>(d_x, rows, K, o, d_scale, d_descale);
            return launch_status();
        }
    }
    // Rows of 2049 to 4096 elements: a workgroup of four wavefronts per row (one 32-byte load per lane) rather than a
    // wavefront per row.  With a wavefront per row every wavefront of an 8192-row tensor is resident at once and all of
    // them read, then all of them write; four times as many, smaller, workgroups come and go in waves, so reads and
    // writes overlap.  Measured inside the benchmark step (input in no cache): 22.5 -> 20.9 us at 8192 x 4096, the same
    // back to back; capping the occupancy of the wavefront-per-row form or giving each wavefront several rows with the
    // next row's loads in flight measured the same or worse.
    if (vec && K > 2 * 1024 && K <= 4 * 1024) k_quant_rows_block<E5M2, 1, GELU><<<rows, kThreads, 0, st>>>(d_x, K, o, d_scale, d_descale);
    else if (vec && K <= 4 * 1024) k_quant_rows<E5M2, 4, GELU><<<grid, kThreads, 0, st>>>(d_x, rows, K, o, d_scale, d_descale);
    else if (vec && K <= 16 * 1024) k_quant_rows_block<E5M2, 4, GELU><<<rows, kThreads, 0, st>>>(d_x, K, o, d_scale, d_descale);
    else if (vec && K <= 32 * 1024) k_quant_rows_block<E5M2, 8, GELU><<<rows, kThreads, 0, st>>>(d_x, K, o, d_scale, d_descale);
    else k_quant_rows_generic<E5M2, GELU><<<rows, kThreads, 0, st>>>(d_x, K, o, d_scale, d_descale);
    return launch_status();
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_fp8_amax_bf16(const uint16_t* d_x, size_t n, float* d_amax, cf_stream_t stream) {
    if (!d_amax || (n > 0 && !d_x)) return CF_ERR_INVALID_ARG;
    // a one-thread fill, not a memset node, so the call can sit inside a captured graph
    k_zero_f32<<<1, 1, 0, as_stream(stream)>>>(d_amax);
    if (n == 0) return launch_status();
    if (aligned16(d_x))
        k_amax_bf16<true><<<min(ceil_div((n + kVec - 1) / kVec, kAmaxThreads), kAmaxBlocks), kAmaxThreads, 0, as_stream(stream)>>>(d_x, n, d_amax);
    else
        k_amax_bf16<false><<<blocks_for(n), kThreads, 0, as_stream(stream)>>>(d_x, n, d_amax);
    return launch_status();
}

int cf_fp8_amax_f32(const float* d_x, size_t n, float* d_amax, cf_stream_t stream) {
    if (!d_amax || (n > 0 && !d_x)) return CF_ERR_INVALID_ARG;
    k_zero_f32<<<1, 1, 0, as_stream(stream)>>>(d_amax);
    if (n == 0) return launch_status();
    const int vec = aligned16(d_x);
    k_amax_f32<<<blocks_for(vec ? (n + 3) / 4 : n), kThreads, 0, as_stream(stream)>>>(d_x, n, d_amax, vec);
    return launch_status();
}

int cf_fp8_scale_from_amax(const float* d_amax, float fp8_max, float* d_scale, float* d_descale,
                           cf_stream_t stream) {
    if (!d_amax || !d_scale || !d_descale) return CF_ERR_INVALID_ARG;
    k_scale_from_amax<<<1, 1, 0, as_stream(stream)>>>(d_amax, fp8_max, d_scale, d_descale);
    return launch_status();
}

int cf_fp8_quantize_e4m3(const uint16_t* d_x, void* d_out, const float* d_scale, size_t n, cf_stream_t stream) {
    return launch_quant<false, false>(d_x, d_out, d_scale, nullptr, n, stream);
}
int cf_fp8_quantize_e5m2(const uint16_t* d_x, void* d_out, const float* d_scale, size_t n, cf_stream_t stream) {
    return launch_quant<true, false>(d_x, d_out, d_scale, nullptr, n, stream);
}
int cf_fp8_quantize_e4m3_record(const uint16_t* d_x, void* d_out, const float* d_scale, float* d_amax,
                                size_t n, cf_stream_t stream) {
    return launch_quant<false, true>(d_x, d_out, d_scale, d_amax, n, stream);
}
int cf_fp8_quantize_e5m2_record(const uint16_t* d_x, void* d_out, const float* d_scale, float* d_amax,
                                size_t n, cf_stream_t stream) {
    return launch_quant<true, true>(d_x, d_out, d_scale, d_amax, n, stream);
}

int cf_fp8_quantize_f32_e4m3(const float* d_x, void* d_out, const float* d_scale, size_t n, cf_stream_t stream) {
    if (n == 0) return CF_OK;
    if (!d_x || !d_out || !d_scale) return CF_ERR_INVALID_ARG;
    const int vec = aligned16(d_x) && (reinterpret_cast<uintptr_t>(d_out) & 3u) == 0;
    k_quant_f32<false><<<blocks_for(vec ? (n + 3) / 4 : n), kThreads, 0, as_stream(stream)>>>(
        d_x, static_cast<uint8_t*>(d_out), d_scale, n, vec);
    return launch_status();
}
int cf_fp8_quantize_f32_e5m2(const float* d_x, void* d_out, const float* d_scale, size_t n, cf_stream_t stream) {
    if (n == 0) return CF_OK;
    if (!d_x || !d_out || !d_scale) return CF_ERR_INVALID_ARG;
    const int vec = aligned16(d_x) && (reinterpret_cast<uintptr_t>(d_out) & 3u) == 0;
    k_quant_f32<true><<<blocks_for(vec ? (n + 3) / 4 : n), kThreads, 0, as_stream(stream)>>>(
        d_x, static_cast<uint8_t*>(d_out), d_scale, n, vec);
    return launch_status();
}

int cf_moe_grouped_quantize_delayed(const uint16_t* d_x, void* d_out, int K, int num_experts, const int* d_counts,
                                    const int* d_offsets, int total_rows, float* d_slot_states, int state_stride_words,
                                    int history_len, int is_e5m2, int apply_gelu, int is_recompute, float* d_row_descale,
                                    cf_stream_t stream) {
    if (K < 0 || num_experts < 0 || total_rows < 0 || history_len < 0) return CF_ERR_INVALID_ARG;
    if (K == 0 || num_experts == 0 || total_rows == 0) return CF_OK;
    if (!d_x || !d_out || !d_counts || !d_offsets || !d_slot_states || !d_row_descale) return CF_ERR_INVALID_ARG;
    if (state_stride_words < cf_act_slot_state_words(history_len)) return CF_ERR_INVALID_ARG;
    if (K % kVec != 0 || !aligned16(d_x) || !aligned16(d_out)) return CF_ERR_UNSUPPORTED;
    // enough workgroups per expert to fill the part, few enough that an expert's arrivals stay a short tail
    unsigned per = 2048u / static_cast<unsigned>(num_experts);
    per = per < 1u ? 1u : (per > 64u ? 64u : per);
    const dim3 grid(per, static_cast<unsigned>(num_experts));
    const float fp8_max = is_e5m2 ? CF_E5M2_MAX : CF_E4M3_MAX;
    hipStream_t st = as_stream(stream);
    auto* o = static_cast<uint8_t*>(d_out);
    auto launch = [&](auto kernel) {
        kernel<<<grid, kThreads, 0, st>>>(d_x, o, K, d_counts, d_offsets, total_rows, d_slot_states, state_stride_words, history_len,
                                          fp8_max, d_row_descale);
    };
    const int which = (is_e5m2 ? 4 : 0) | (apply_gelu ? 2 : 0) | (is_recompute ? 1 : 0);
    // GELU over a large bank: the table form (the direct form waits for erff, about 40 vector instructions per element)
    if (apply_gelu && num_experts <= kLutMaxExperts && static_cast<size_t>(total_rows) * K >= (64u << 20)) {
        static std::once_flag once;
        static hipError_t err = hipSuccess;
        static int cus = 256;
        std::call_once(once, [] {
            const void* ks[4] = {reinterpret_cast<const void*>(&k_grouped_gelu_quant_delayed_lut<false, false>),
                                 reinterpret_cast<const void*>(&k_grouped_gelu_quant_delayed_lut<false, true>),
                                 reinterpret_cast<const void*>(&k_grouped_gelu_quant_delayed_lut<true, false>),
                                 reinterpret_cast<const void*>(&k_grouped_gelu_quant_delayed_lut<true, true>)};
            for (const void* k : ks) {
                const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
                if (e != hipSuccess) err = e;
            }
            int dev = 0, n = 0;
            if (hipGetDevice(&dev) == hipSuccess &&
                hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
                cus = n;
        });
        if (err != hipSuccess) return static_cast<int>(err);
        // parts per expert: about four items per resident workgroup, so ragged experts even out
        int parts = (4 * cus + num_experts - 1) / num_experts;
        parts = parts < 1 ? 1 : (parts > 64 ? 64 : parts);
        auto launch_lut = [&](auto kernel) {
            kernel<<<cus, kLutThreads, 128 * 1024, st>>>(d_x, o, K, d_counts, d_offsets, total_rows, num_experts, parts, d_slot_states,
                                                         state_stride_words, history_len, fp8_max, d_row_descale);
        };
        switch (which & 5) {
            case 0: launch_lut(k_grouped_gelu_quant_delayed_lut<false, false>); break;
            case 1: launch_lut(k_grouped_gelu_quant_delayed_lut<false, true>); break;
            case 4: launch_lut(k_grouped_gelu_quant_delayed_lut<true, false>); break;
            default: launch_lut(k_grouped_gelu_quant_delayed_lut<true, true>); break;
        }
        return launch_status();
    }
    switch (which) {
        case 0: launch(k_grouped_quant_delayed<false, false, false>); break;
        case 1: launch(k_grouped_quant_delayed<false, false, true>); break;
        case 2: launch(k_grouped_quant_delayed<false, true, false>); break;
        case 3: launch(k_grouped_quant_delayed<false, true, true>); break;
        case 4: launch(k_grouped_quant_delayed<true, false, false>); break;
        case 5: launch(k_grouped_quant_delayed<true, false, true>); break;
        case 6: launch(k_grouped_quant_delayed<true, true, false>); break;
        default: launch(k_grouped_quant_delayed<true, true, true>); break;
    }
    return launch_status();
}

int cf_fp8_quantize_delayed_step(const uint16_t* d_x, void* d_out, size_t n, int is_e5m2, float* d_amax, float* d_scale,
                                 float* d_descale, float* d_scale_snapshot, float* d_descale_snapshot, float* d_history,
                                 int history_len, int* d_history_cursor, int* d_history_count, float* d_running_amax,
                                 unsigned int* d_arrived, cf_stream_t stream) {
    if (!d_amax || !d_scale || !d_descale || !d_scale_snapshot || !d_descale_snapshot || !d_running_amax || !d_arrived ||
        history_len < 0 || (history_len > 0 && (!d_history || !d_history_cursor || !d_history_count)) ||
        (n > 0 && (!d_x || !d_out)))
        return CF_ERR_INVALID_ARG;
    DelayedStep d{d_amax, d_scale, d_descale, d_scale_snapshot, d_descale_snapshot, d_history, history_len,
                  d_history_cursor, d_history_count, d_running_amax, d_arrived, is_e5m2 ? CF_E5M2_MAX : CF_E4M3_MAX};
    auto* o = static_cast<uint8_t*>(d_out);
    hipStream_t st = as_stream(stream);
    // n == 0 still runs one workgroup: the state advances with an amax of zero, as the separate launches would
    auto grid_for = [](size_t items) { return max(1u, min(ceil_div(items, kAmaxThreads), kAmaxBlocks)); };
    if (aligned16(d_x) && aligned16(d_out)) {
        const unsigned grid = grid_for((n + kVec - 1) / kVec);
        if (is_e5m2) k_quant_delayed_step<true, true><<<grid, kAmaxThreads, 0, st>>>(d_x, o, n, d);
        else         k_quant_delayed_step<false, true><<<grid, kAmaxThreads, 0, st>>>(d_x, o, n, d);
    } else {
        const unsigned grid = grid_for(n);
        if (is_e5m2) k_quant_delayed_step<true, false><<<grid, kAmaxThreads, 0, st>>>(d_x, o, n, d);
        else         k_quant_delayed_step<false, false><<<grid, kAmaxThreads, 0, st>>>(d_x, o, n, d);
    }
    return launch_status();
}

int cf_fp8_update_delayed_scale(const float* d_amax, float fp8_max, float* d_scale, float* d_descale,
                                float* d_history, int history_len, int* d_history_cursor,
                                int* d_history_count, cf_stream_t stream) {
    if (!d_amax || !d_scale || !d_descale) return CF_ERR_INVALID_ARG;
    if (history_len > 0 && (!d_history || !d_history_cursor || !d_history_count)) return CF_ERR_INVALID_ARG;
    k_update_delayed_scale<<<1, 1, 0, as_stream(stream)>>>(d_amax, fp8_max, d_scale, d_descale, d_history,
                                                           history_len, d_history_cursor, d_history_count);
    return launch_status();
}

int cf_fp8_clip_probe(const float* d_amax, const float* d_scale, float fp8_max, float* d_stats,
                      cf_stream_t stream) {
    if (!d_amax || !d_scale || !d_stats) return CF_ERR_INVALID_ARG;
    k_clip_probe<<<1, 1, 0, as_stream(stream)>>>(d_amax, d_scale, fp8_max, d_stats);
    return launch_status();
}

int cf_fp8_elem_clip_count(const uint16_t* d_x, const float* d_scale, float fp8_max, size_t n, float* d_out,
                           cf_stream_t stream) {
    if (!d_scale || !d_out || (n > 0 && !d_x)) return CF_ERR_INVALID_ARG;
    k_elem_clip_count<<<blocks_for(n), kThreads, 0, as_stream(stream)>>>(d_x, d_scale, fp8_max, n, d_out);
    return launch_status();
}

int cf_fp8_calib_minmax_update(const float* d_amax, float* d_cmin, float* d_cmax, cf_stream_t stream) {
    if (!d_amax || !d_cmin || !d_cmax) return CF_ERR_INVALID_ARG;
    k_calib_minmax<<<1, 1, 0, as_stream(stream)>>>(d_amax, d_cmin, d_cmax);
    return launch_status();
}

int cf_fp8_quantize_rows(const uint16_t* d_x, int rows, int K, int is_e5m2, void* d_out, float* d_scale,
                         float* d_descale, cf_stream_t stream) {
    return is_e5m2 ? launch_quant_rows<true, false>(d_x, rows, K, d_out, d_scale, d_descale, stream)
                   : launch_quant_rows<false, false>(d_x, rows, K, d_out, d_scale, d_descale, stream);
}

int cf_gelu_quantize_rows_e4m3(const uint16_t* d_x, int rows, int K, void* d_out, float* d_scale, float* d_descale,
                               cf_stream_t stream) {
    return launch_quant_rows<false, true>(d_x, rows, K, d_out, d_scale, d_descale, stream);
}

int cf_fp8_quantize_block_1x128(const uint16_t* d_x, int rows, int K, void* d_out, float* d_scale,
                                float* d_descale, cf_stream_t stream) {
    if (rows < 0 || K < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || K == 0) return CF_OK;
    if (!d_x || !d_out || !d_scale || !d_descale) return CF_ERR_INVALID_ARG;
    auto* o = static_cast<uint8_t*>(d_out);
    if (K % 128 == 0 && aligned16(d_x) && aligned16(d_out)) {
        const size_t ngroups = static_cast<size_t>(rows) * (K / 128);
        k_quant_1x128<<<blocks_for(ngroups * 8), kThreads, 0, as_stream(stream)>>>(d_x, ngroups, o, d_scale, d_descale);
    } else {
        const size_t ngroups = static_cast<size_t>(rows) * ((K + 127) / 128);
        k_quant_1x128_generic<<<ceil_div(ngroups, kThreads / 64), kThreads, 0, as_stream(stream)>>>(
            d_x, rows, K, o, d_scale, d_descale);
    }
    return launch_status();
}

int cf_fp8_quantize_block_128x128(const uint16_t* d_x, int rows, int K, void* d_out, float* d_scale,
                                  float* d_descale, cf_stream_t stream) {
    if (rows < 0 || K < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || K == 0) return CF_OK;
    if (!d_x || !d_out || !d_scale || !d_descale) return CF_ERR_INVALID_ARG;
    const int vec = K % 128 == 0 && aligned16(d_x) && aligned16(d_out);
    const unsigned grid = static_cast<unsigned>(((rows + 127) / 128) * ((K + 127) / 128));
    k_quant_128x128<<<grid, kThreads, 0, as_stream(stream)>>>(d_x, rows, K, static_cast<uint8_t*>(d_out),
                                                              d_scale, d_descale, vec);
    return launch_status();
}

int cf_fp8_pack_bf16_e4m3_raw(const uint16_t* d_x, uint8_t* d_out, float* d_amax, float* d_scale,
                              float* d_descale, int* d_bad_count, size_t n, cf_stream_t stream) {
    if (!d_amax || !d_scale || !d_descale || !d_bad_count || (n > 0 && (!d_x || !d_out))) return CF_ERR_INVALID_ARG;
    hipStream_t st = as_stream(stream);
    k_zero_raw<<<1, 1, 0, st>>>(d_amax, d_bad_count);
    if (n) k_raw_stats<<<blocks_for(n), kThreads, 0, st>>>(d_x, n, d_amax, d_bad_count);
    k_scale_from_amax<<<1, 1, 0, st>>>(d_amax, 448.0f, d_scale, d_descale);
    if (n) k_raw_pack<false><<<blocks_for(n), kThreads, 0, st>>>(d_x, d_out, nullptr, d_scale, d_descale, d_bad_count, n);
    return launch_status();
}

int cf_fp8_pack_bf16_e4m3_raw_and_dequant(const uint16_t* d_x, uint8_t* d_out, uint16_t* d_dequant,
                                          float* d_amax, float* d_scale, float* d_descale,
                                          int* d_bad_count, size_t n, cf_stream_t stream) {
    if (!d_amax || !d_scale || !d_descale || !d_bad_count || (n > 0 && (!d_x || !d_out || !d_dequant)))
        return CF_ERR_INVALID_ARG;
    hipStream_t st = as_stream(stream);
    k_zero_raw<<<1, 1, 0, st>>>(d_amax, d_bad_count);
    if (n) k_raw_stats<<<blocks_for(n), kThreads, 0, st>>>(d_x, n, d_amax, d_bad_count);
    k_scale_from_amax<<<1, 1, 0, st>>>(d_amax, 448.0f, d_scale, d_descale);
    if (n) k_raw_pack<true><<<blocks_for(n), kThreads, 0, st>>>(d_x, d_out, d_dequant, d_scale, d_descale, d_bad_count, n);
    return launch_status();
}

int cf_fp8_unpack_e4m3_raw_bf16(const uint8_t* d_in, const float* d_descale, uint16_t* d_out, size_t n,
                                cf_stream_t stream) {
    if (n == 0) return CF_OK;
    if (!d_in || !d_descale || !d_out) return CF_ERR_INVALID_ARG;
    k_raw_unpack<<<blocks_for(n), kThreads, 0, as_stream(stream)>>>(d_in, d_descale, d_out, n);
    return launch_status();
}

}  // extern "C"
