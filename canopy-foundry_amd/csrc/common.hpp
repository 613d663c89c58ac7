// Shared device helpers for the gfx950 FP8 kernels: bf16 <-> f32, OCP fp8
// encode/decode, wavefront (64-lane) reductions, launch bookkeeping.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cf_fp8.h"

#ifndef __gfx950__
#if defined(__HIP_DEVICE_COMPILE__)
#error "this library is written for gfx950 (MI355X) only"
#endif
#endif

namespace cf {

constexpr int kWave = 64;

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// Round-to-nearest-even, NaN kept quiet.
__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
    const uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((bits >> 16) | 0x0040u);
    return static_cast<uint16_t>((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}

// Streaming stores: 16 or 8 bytes that this kernel does not read again.  Marked non-temporal, they leave through the
// L2 without taking lines from the data that is read; on write-heavy kernels (a dual quantize writes as many bytes as
// it reads) this is worth 30 % of the run time.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_stream16(void* p, uint4 v) {
    const u32x4_t vv = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(vv, static_cast<u32x4_t*>(p));
}
__device__ __forceinline__ void store_stream8(void* p, uint2 v) {
    const u32x2_t vv = {v.x, v.y};
    __builtin_nontemporal_store(vv, static_cast<u32x2_t*>(p));
}

// Exact-erf GELU in fp32 (gelu_forward_kernel, kernels/moe.cu:510-517 of the reference), and the same on a packed bf16 pair with
// one rounding of each result to bf16.
__device__ __forceinline__ float gelu_fwd(float v) { return 0.5f * v * (1.0f + erff(v * 0.7071067811865476f)); }
__device__ __forceinline__ uint32_t gelu2(uint32_t pair) { return pack_bf16x2(gelu_fwd(bf16_lo(pair)), gelu_fwd(bf16_hi(pair))); }

// Two floats -> packed bf16 pair on gfx950's v_cvt_pk_bf16_f32 (round to nearest even).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2_hw(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float round_bf16_hw(float v) { return __uint_as_float(pack_bf16x2_hw(v, 0.0f) << 16); }

// ---- OCP fp8 encode -------------------------------------------------------
// gfx950's v_cvt_pk_{fp8,bf8}_f32 round to nearest even onto OCP e4m3fn / e5m2.
// Saturation to the largest finite value is applied here by clamping first
// (v_med3_f32); NaN is restored afterwards as sign|0x7f.
template <bool E5M2>
__device__ __forceinline__ float fp8_clamp(float v) {
    constexpr float m = E5M2 ? 57344.0f : 448.0f;
    return __builtin_amdgcn_fmed3f(v, -m, m);
}
__device__ __forceinline__ uint32_t nan_fix(uint32_t packed, float v, int byte) {
    if (v != v) {
        const uint32_t code = ((__float_as_uint(v) >> 24) & 0x80u) | 0x7fu;
        packed = (packed & ~(0xffu << (8 * byte))) | (code << (8 * byte));
    }
    return packed;
}
// four floats -> four fp8 bytes, byte i holds v_i
template <bool E5M2>
__device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
    int r = 0;
    if constexpr (E5M2) {
        r = __builtin_amdgcn_cvt_pk_bf8_f32(fp8_clamp<true>(a), fp8_clamp<true>(b), r, false);
        r = __builtin_amdgcn_cvt_pk_bf8_f32(fp8_clamp<true>(c), fp8_clamp<true>(d), r, true);
    } else {
        r = __builtin_amdgcn_cvt_pk_fp8_f32(fp8_clamp<false>(a), fp8_clamp<false>(b), r, false);
        r = __builtin_amdgcn_cvt_pk_fp8_f32(fp8_clamp<false>(c), fp8_clamp<false>(d), r, true);
    }
    uint32_t u = static_cast<uint32_t>(r);
    u = nan_fix(u, a, 0); u = nan_fix(u, b, 1); u = nan_fix(u, c, 2); u = nan_fix(u, d, 3);
    return u;
}
// the same for inputs known to hold no NaN
template <bool E5M2>
__device__ __forceinline__ uint32_t cvt4_fp8_finite(float a, float b, float c, float d) {
    int r = 0;
    if constexpr (E5M2) {
        r = __builtin_amdgcn_cvt_pk_bf8_f32(fp8_clamp<true>(a), fp8_clamp<true>(b), r, false);
        r = __builtin_amdgcn_cvt_pk_bf8_f32(fp8_clamp<true>(c), fp8_clamp<true>(d), r, true);
    } else {
        r = __builtin_amdgcn_cvt_pk_fp8_f32(fp8_clamp<false>(a), fp8_clamp<false>(b), r, false);
        r = __builtin_amdgcn_cvt_pk_fp8_f32(fp8_clamp<false>(c), fp8_clamp<false>(d), r, true);
    }
    return static_cast<uint32_t>(r);
}
template <bool E5M2>
__device__ __forceinline__ uint8_t cvt1_fp8(float a) {
    return static_cast<uint8_t>(cvt4_fp8<E5M2>(a, 0.0f, 0.0f, 0.0f) & 0xffu);
}

// ---- fp8 decode (exact) -----------------------------------------------------
__device__ __forceinline__ float e4m3_to_f32(uint8_t b) {
    const uint32_t sign = (static_cast<uint32_t>(b) & 0x80u) << 24;
    const uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    float mag;
    if (e == 0) mag = static_cast<float>(m) * 0.001953125f;           // m * 2^-9
    else if (e == 15 && m == 7) return __uint_as_float(0x7fc00000u);   // one NaN for both signs, as unpack() does
    else mag = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return __uint_as_float(__float_as_uint(mag) | sign);
}
__device__ __forceinline__ float e5m2_to_f32(uint8_t b) {
    const uint32_t sign = (static_cast<uint32_t>(b) & 0x80u) << 24;
    const uint32_t e = (b >> 2) & 0x1fu, m = b & 3u;
    float mag;
    if (e == 0) mag = static_cast<float>(m) * 1.52587890625e-05f;     // m * 2^-16
    else if (e == 31 && m != 0) return __uint_as_float(0x7fc00000u);
    else if (e == 31) mag = __uint_as_float(0x7f800000u);
    else mag = __uint_as_float(((e + 112u) << 23) | (m << 21));
    return __uint_as_float(__float_as_uint(mag) | sign);
}

// ---- 64-lane wavefront reductions ------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Running maximum of |bf16| over both halves of packed pairs, as integers (|x| orders like its bits; any NaN
// ends up above the infinity pattern 0x7f80)
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_absmax(uint32_t acc, uint32_t pair) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, acc),
                                                                  __builtin_bit_cast(u16x2, pair & 0x7fff7fffu)));
}

// The 64-lane maximum of such an accumulator as bf16 bits: below 0x7f80 every element was finite.
__device__ __forceinline__ int wave_absmax_bits(uint32_t acc) {
    int m = static_cast<int>(max(acc & 0xffffu, acc >> 16));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off, kWave));
    return m;
}

// |x| >= 0 orders like its bit pattern, so an integer max is a float max.  Thousands of atomics on one
// address serialise in L2 (about 13 ns each), so the value is read first and the atomic is issued only by a
// caller that would raise it: the running maximum settles after a handful of updates, and a stale read
// merely costs a redundant atomic.
__device__ __forceinline__ void atomic_max_nonneg(float* addr, float v) {
    int* p = reinterpret_cast<int*>(addr);
    if (__float_as_int(v) > __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(p, __float_as_int(v));
}

// "Last workgroup in" without an agent-scope fence.  A release fence at agent scope writes the XCD's whole L2 back
// (the eight L2s are not coherent with each other) and waits for every store the wavefront has in flight: measured at
// 15 us per workgroup under a streaming kernel.  What the pattern needs is less: that a workgroup's maximum is in place
// before its arrival counts.  Agent-scope atomics are performed at the memory side, past the L2s; the maximum is issued
// with its return value taken, and the arrival's operand depends on that value, so the arrival cannot be issued before
// the maximum has been performed.  A workgroup that would not raise the maximum has nothing to publish: the value it
// read came from an atomic that has been performed.  The caller that gets `true` arrived last of `expected`; every
// other arrival, and with it every maximum, has been performed by then, and it reads the result with
// atomic_load_agent().  Values are non-negative floats, which order like their bit patterns.
__device__ __forceinline__ bool arrive_with_max(float* running, unsigned* arrived, float v, unsigned expected) {
    int* p = reinterpret_cast<int*>(running);
    unsigned one = 1u;
    if (__float_as_int(v) > __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
        int old = __hip_atomic_fetch_max(p, __float_as_int(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("" : "+v"(old) : : "memory");
        one += static_cast<unsigned>(old) >> 31;             // old is a non-negative float's bits: adds nothing
    }
    const unsigned before = __hip_atomic_fetch_add(arrived, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("" : : : "memory");
    return before == expected - 1u;
}
__device__ __forceinline__ float atomic_load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- deterministic expf ------------------------------------------------------
// Cody-Waite reduction + degree-6 polynomial with explicit FMAs and exact
// power-of-two scaling.  Uses only IEEE-exact operations so that a host
// restatement of the same steps yields the same bits.
__device__ __forceinline__ float det_expf(float x) {
    if (x != x) return x;
    if (x > 88.72284f) return __uint_as_float(0x7f800000u);
    if (x < -103.97208f) return 0.0f;
    const float k = __builtin_rintf(x * 1.44269504f);
    float r = __builtin_fmaf(k, -0.693359375f, x);
    r = __builtin_fmaf(k, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    p = __builtin_fmaf(p, r * r, r);
    p = p + 1.0f;
    const int ki = static_cast<int>(k);
    if (ki < -126) return (p * __uint_as_float(static_cast<uint32_t>(ki + 227) << 23)) * 7.8886090522101181e-31f;
    if (ki > 127) return (p * __uint_as_float(static_cast<uint32_t>(ki + 126) << 23)) * 2.0f;
    return p * __uint_as_float(static_cast<uint32_t>(ki + 127) << 23);
}
// 1 / (1 + e^-x) for x >= 0, e^x / (1 + e^x) below: one exponential of -|x| and one division serve both
__device__ __forceinline__ float stable_sigmoid(float x) {
    const float e = det_expf(-fabsf(x));
    return (x >= 0.0f ? 1.0f : e) / (1.0f + e);
}

// ---- host-side launch helpers ----------------------------------------------
// Every entry point converts its stream argument before it launches anything; that is also where an
// error left behind by an earlier, unrelated runtime call of the process (an event query that was not
// ready, say) is discarded, so that launch_status() reports this library's launches only.
inline hipStream_t as_stream(cf_stream_t s) {
    (void)hipGetLastError();
    return static_cast<hipStream_t>(s);
}
inline int launch_status() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? CF_OK : static_cast<int>(e);
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline unsigned ceil_div(size_t a, size_t b) { return static_cast<unsigned>((a + b - 1) / b); }

}  // namespace cf
