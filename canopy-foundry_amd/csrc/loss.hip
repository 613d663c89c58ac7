// Chunked cross-entropy forward + backward over bf16 logits, optionally fused with the E5M2 recording quantize
// of the gradient that the FP8 head's input-gradient GEMM consumes.
//
// The reference (kernels/cross_entropy.cu:201-305) runs one 128-thread block per row that reads the row three
// times (max, sum of exp, gradient); the FP8 path then reads the bf16 gradient once more to quantize it
// (src/trainer.cu:8053-8058).  Here a 256-lane workgroup keeps a row of up to 32768 logits in registers (a 1024-lane
// one a row of up to 131072): HBM
// sees 2 B read + 2 B (bf16 gradient, which the weight-gradient GEMM needs) + 1 B (E5M2) written per element.
//
// exp and log run on the hardware exp2 / log2 units (about 1 ulp; CUDA's expf / logf bits cannot be reproduced
// anyway), so the gradient is within one bf16 ulp of the correctly rounded value rather than bit-defined;
// the E5M2 bytes are the exact quantization of the bf16 gradient this kernel writes.
#include "common.hpp"

namespace cf {
namespace {

constexpr int kCeThreads = 256;
constexpr int kCeWide = 1024;                          // lanes per row for rows beyond 32768 logits
constexpr int kCeMaxChunks = 16;                       // 8-element chunks per lane: rows up to 32768 logits
constexpr float kLog2e = 1.44269504088896340736f, kLn2 = 0.69314718055994530942f;

struct CeArgs {
    const uint16_t* logits; const int32_t* labels; float* loss; uint16_t* grad; const int* n_valid;
    uint8_t* grad8; const float* qscale; float* amax;   // QUANT only
    int V;
};

__device__ __forceinline__ float block_reduce(float v, float* sh, bool is_max) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off, kWave);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    __syncthreads();                       // sh may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = sh[0];
    for (int w = 1; w < static_cast<int>(blockDim.x >> 6); ++w) r = is_max ? fmaxf(r, sh[w]) : r + sh[w];
    return r;
}

__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

// one gradient element: kernels/cross_entropy.cu:263-268
__device__ __forceinline__ float ce_grad(float logit, float row_max, float inv_sum, float inv_n, bool is_label, float& label_log_prob) {
    const float prob = fast_exp(logit - row_max) * inv_sum;
    if (is_label) label_log_prob = __builtin_amdgcn_logf(prob + 1e-9f) * kLn2;
    return (prob - (is_label ? 1.0f : 0.0f)) * inv_n;
}

// The chunk's four words as the compiler cannot relate to their earlier uses: without this it unpacks all 128
// logits of a lane to fp32 once and keeps them live across the three passes (184 registers, two wavefronts per
// SIMD); unpacking again in each pass costs one instruction per element and halves the register count.
__device__ __forceinline__ void opaque_words(const uint4& v, uint32_t (&w)[4]) {
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    asm volatile("" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]));
}

// Row in registers: V % 8 == 0, V <= 128 T, 16-byte aligned rows (8-byte for the fp8 gradient).  T lanes per row: 256
// for rows up to 32768 logits, 1024 (a CU's sixteen wavefronts, 128 registers each) for rows up to 131072, so that a
// 128k vocabulary is still read from memory once.
template <bool QUANT, int T>
__global__ __launch_bounds__(T) void k_ce_rows(const CeArgs p) {
    __shared__ float sh[T / 64];
    const int tid = threadIdx.x, V = p.V, nchunks = V / 8;
    const size_t row = blockIdx.x;
    const int label = p.labels[row];
    uint16_t* grow = p.grad + row * V;
    uint8_t* qrow = QUANT ? p.grad8 + row * V : nullptr;
    if (label < 0) {                                     // ignored token: zero gradient, no loss (:237-241)
        for (int c = tid; c < nchunks; c += T) {
            reinterpret_cast<uint4*>(grow)[c] = make_uint4(0, 0, 0, 0);
            if constexpr (QUANT) reinterpret_cast<uint2*>(qrow)[c] = make_uint2(0, 0);
        }
        return;
    }
    const uint16_t* lrow = p.logits + row * V;
    uint4 v[kCeMaxChunks];
    float m = -3.402823466e38f;
#pragma unroll
    for (int j = 0; j < kCeMaxChunks; ++j) {
        const int c = tid + j * T;
        if (c < nchunks) {
            v[j] = reinterpret_cast<const uint4*>(lrow)[c];
            const uint32_t w[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int k = 0; k < 4; ++k) m = fmaxf(m, fmaxf(bf16_lo(w[k]), bf16_hi(w[k])));
        }
    }
    const float row_max = block_reduce(m, sh, true);
    // exp(x - max) as exp2(x * log2e - max * log2e): one fused multiply-add per element feeds the exp2 unit
    const float bias2 = -row_max * kLog2e;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < kCeMaxChunks; ++j) {
        if (tid + j * T < nchunks) {
            uint32_t w[4];
            opaque_words(v[j], w);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                s += __builtin_amdgcn_exp2f(__builtin_fmaf(bf16_lo(w[k]), kLog2e, bias2)) +
                     __builtin_amdgcn_exp2f(__builtin_fmaf(bf16_hi(w[k]), kLog2e, bias2));
        }
        __builtin_amdgcn_sched_barrier(0);       // one chunk's temporaries at a time: the row itself takes 64 registers
    }
    const float inv_sum = 1.0f / block_reduce(s, sh, false);
    const float inv_n = 1.0f / static_cast<float>(max(*p.n_valid, 1));
    const float both = inv_sum * inv_n;                  // every column but the label's: exp * (1 / sum) * (1 / n)
    const float qs = QUANT ? *p.qscale : 0.0f;
    const bool qs_finite = fabsf(qs) < __uint_as_float(0x7f800000u);
    const int label_chunk = label >> 3;
    float llp = 0.0f;
    uint32_t absacc = 0;
#pragma unroll
    for (int j = 0; j < kCeMaxChunks; ++j) {
        const int c = tid + j * T;
        if (c < nchunks) {
            uint32_t w[4];
            opaque_words(v[j], w);
            uint32_t o[4];
            if (c != label_chunk) {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    o[k] = pack_bf16x2_hw(__builtin_amdgcn_exp2f(__builtin_fmaf(bf16_lo(w[k]), kLog2e, bias2)) * both,
                                          __builtin_amdgcn_exp2f(__builtin_fmaf(bf16_hi(w[k]), kLog2e, bias2)) * both);
            } else {
                // the chunk with the label's column: kernels/cross_entropy.cu:263-268 as written
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int e = c * 8 + 2 * k;
                    o[k] = pack_bf16x2_hw(ce_grad(bf16_lo(w[k]), row_max, inv_sum, inv_n, e == label, llp),
                                          ce_grad(bf16_hi(w[k]), row_max, inv_sum, inv_n, e + 1 == label, llp));
                }
            }
            store_stream16(reinterpret_cast<uint4*>(grow) + c, make_uint4(o[0], o[1], o[2], o[3]));
            if constexpr (QUANT) {
                // src/trainer.cu:8053: the E5M2 quantize of the bf16 gradient with the slot's previous scale, amax recorded
                const uint32_t acc8 = pk_absmax(pk_absmax(pk_absmax(pk_absmax(0u, o[0]), o[1]), o[2]), o[3]);
                absacc = pk_absmax(absacc, acc8);        // sign bits are clear in both
                uint2 q;
                if (max(acc8 & 0xffffu, acc8 >> 16) < 0x7f80u && qs_finite) {
                    q.x = cvt4_fp8_finite<true>(bf16_lo(o[0]) * qs, bf16_hi(o[0]) * qs, bf16_lo(o[1]) * qs, bf16_hi(o[1]) * qs);
                    q.y = cvt4_fp8_finite<true>(bf16_lo(o[2]) * qs, bf16_hi(o[2]) * qs, bf16_lo(o[3]) * qs, bf16_hi(o[3]) * qs);
                } else {
                    q.x = cvt4_fp8<true>(bf16_lo(o[0]) * qs, bf16_hi(o[0]) * qs, bf16_lo(o[1]) * qs, bf16_hi(o[1]) * qs);
                    q.y = cvt4_fp8<true>(bf16_lo(o[2]) * qs, bf16_hi(o[2]) * qs, bf16_lo(o[3]) * qs, bf16_hi(o[3]) * qs);
                }
                reinterpret_cast<uint2*>(qrow)[c] = q;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    // only the lane that met the label holds a non-zero term (:269-272)
    const float g_llp = block_reduce(llp, sh, false);
    if (tid == 0) atomicAdd(p.loss, -g_llp * inv_n);
    if constexpr (QUANT) {
        // gradients are finite or NaN, never larger than 2: the bit maximum is the float maximum unless a NaN is present,
        // and a NaN gradient row leaves the recorded amax to the finite rows, as a float maximum would
        int mb = wave_absmax_bits(absacc);
        if (mb > 0x7f80) mb = 0;
        const float a = block_reduce(__uint_as_float(static_cast<uint32_t>(mb) << 16), sh, true);
        if (tid == 0) atomic_max_nonneg(p.amax, a);
    }
}

// Rows longer than the register-resident form takes (V % 8 == 0, aligned): the same arithmetic with the row read
// three times in 16-byte vectors; the second and third reads mostly come from the caches.
template <bool QUANT>
__global__ __launch_bounds__(kCeThreads) void k_ce_rows_stream(const CeArgs p) {
    __shared__ float sh[kCeThreads / 64];
    const int tid = threadIdx.x, V = p.V, nchunks = V / 8;
    const size_t row = blockIdx.x;
    const int label = p.labels[row];
    uint16_t* grow = p.grad + row * V;
    uint8_t* qrow = QUANT ? p.grad8 + row * V : nullptr;
    if (label < 0) {
        for (int c = tid; c < nchunks; c += kCeThreads) {
            reinterpret_cast<uint4*>(grow)[c] = make_uint4(0, 0, 0, 0);
            if constexpr (QUANT) reinterpret_cast<uint2*>(qrow)[c] = make_uint2(0, 0);
        }
        return;
    }
    const uint4* lrow = reinterpret_cast<const uint4*>(p.logits + row * V);
    float m = -3.402823466e38f;
    for (int c = tid; c < nchunks; c += kCeThreads) {
        const uint4 v = lrow[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) m = fmaxf(m, fmaxf(bf16_lo(w[k]), bf16_hi(w[k])));
    }
    const float row_max = block_reduce(m, sh, true);
    const float bias2 = -row_max * kLog2e;
    float s = 0.0f;
    for (int c = tid; c < nchunks; c += kCeThreads) {
        const uint4 v = lrow[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            s += __builtin_amdgcn_exp2f(__builtin_fmaf(bf16_lo(w[k]), kLog2e, bias2)) +
                 __builtin_amdgcn_exp2f(__builtin_fmaf(bf16_hi(w[k]), kLog2e, bias2));
    }
    const float inv_sum = 1.0f / block_reduce(s, sh, false);
    const float inv_n = 1.0f / static_cast<float>(max(*p.n_valid, 1));
    const float both = inv_sum * inv_n;
    const float qs = QUANT ? *p.qscale : 0.0f;
    const int label_chunk = label >> 3;
    float llp = 0.0f;
    uint32_t absacc = 0;
    for (int c = tid; c < nchunks; c += kCeThreads) {
        const uint4 v = lrow[c];                           // read before the (possibly aliasing) store below
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
        if (c != label_chunk) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                o[k] = pack_bf16x2_hw(__builtin_amdgcn_exp2f(__builtin_fmaf(bf16_lo(w[k]), kLog2e, bias2)) * both,
                                      __builtin_amdgcn_exp2f(__builtin_fmaf(bf16_hi(w[k]), kLog2e, bias2)) * both);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int e = c * 8 + 2 * k;
                o[k] = pack_bf16x2_hw(ce_grad(bf16_lo(w[k]), row_max, inv_sum, inv_n, e == label, llp),
                                      ce_grad(bf16_hi(w[k]), row_max, inv_sum, inv_n, e + 1 == label, llp));
            }
        }
        store_stream16(reinterpret_cast<uint4*>(grow) + c, make_uint4(o[0], o[1], o[2], o[3]));
        if constexpr (QUANT) {
            absacc = pk_absmax(pk_absmax(pk_absmax(pk_absmax(absacc, o[0]), o[1]), o[2]), o[3]);
            uint2 q;
            q.x = cvt4_fp8<true>(bf16_lo(o[0]) * qs, bf16_hi(o[0]) * qs, bf16_lo(o[1]) * qs, bf16_hi(o[1]) * qs);
            q.y = cvt4_fp8<true>(bf16_lo(o[2]) * qs, bf16_hi(o[2]) * qs, bf16_lo(o[3]) * qs, bf16_hi(o[3]) * qs);
            reinterpret_cast<uint2*>(qrow)[c] = q;
        }
    }
    const float g_llp = block_reduce(llp, sh, false);
    if (tid == 0) atomicAdd(p.loss, -g_llp * inv_n);
    if constexpr (QUANT) {
        int mb = wave_absmax_bits(absacc);
        if (mb > 0x7f80) mb = 0;                           // a NaN row leaves the recorded amax to the finite rows
        const float a = block_reduce(__uint_as_float(static_cast<uint32_t>(mb) << 16), sh, true);
        if (tid == 0) atomic_max_nonneg(p.amax, a);
    }
}

// Any V, any alignment: three passes over the row, as the reference does.
template <bool QUANT>
__global__ __launch_bounds__(kCeThreads) void k_ce_rows_generic(const CeArgs p) {
    __shared__ float sh[kCeThreads / 64];
    const int tid = threadIdx.x, V = p.V;
    const size_t row = blockIdx.x;
    const int label = p.labels[row];
    uint16_t* grow = p.grad + row * V;
    uint8_t* qrow = QUANT ? p.grad8 + row * V : nullptr;
    if (label < 0) {
        for (int i = tid; i < V; i += kCeThreads) {
            grow[i] = 0;
            if constexpr (QUANT) qrow[i] = 0;
        }
        return;
    }
    const uint16_t* lrow = p.logits + row * V;
    float m = -3.402823466e38f;
    for (int i = tid; i < V; i += kCeThreads) m = fmaxf(m, bf16_to_f32(lrow[i]));
    const float row_max = block_reduce(m, sh, true);
    float s = 0.0f;
    for (int i = tid; i < V; i += kCeThreads) s += fast_exp(bf16_to_f32(lrow[i]) - row_max);
    const float inv_sum = 1.0f / block_reduce(s, sh, false);
    const float inv_n = 1.0f / static_cast<float>(max(*p.n_valid, 1));
    const float qs = QUANT ? *p.qscale : 0.0f;
    float llp = 0.0f, amax = 0.0f;
    for (int i = tid; i < V; i += kCeThreads) {
        const uint16_t g = f32_to_bf16(ce_grad(bf16_to_f32(lrow[i]), row_max, inv_sum, inv_n, i == label, llp));
        grow[i] = g;                                     // may alias lrow[i]: read above, never read again
        if constexpr (QUANT) {
            const float gf = bf16_to_f32(g);
            amax = fmaxf(amax, fabsf(gf));
            qrow[i] = cvt1_fp8<true>(gf * qs);
        }
    }
    const float g_llp = block_reduce(llp, sh, false);
    if (tid == 0) atomicAdd(p.loss, -g_llp * inv_n);
    if constexpr (QUANT) {
        const float a = block_reduce(amax, sh, true);
        if (tid == 0) atomic_max_nonneg(p.amax, a);
    }
}

// kernels/cross_entropy.cu:201-219
__global__ __launch_bounds__(kCeThreads) void k_count_valid(const int32_t* __restrict__ labels, int n, int* __restrict__ n_valid) {
    int local = 0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) local += labels[i] >= 0 ? 1 : 0;
    local = wave_sum_i(local);
    if ((threadIdx.x & 63) == 0 && local) atomicAdd(n_valid, local);
}

template <bool QUANT>
int launch_ce(const CeArgs& p, int rows, hipStream_t st) {
    const bool vec = p.V % 8 == 0 && aligned16(p.logits) && aligned16(p.grad) &&
                     (!QUANT || (reinterpret_cast<uintptr_t>(p.grad8) & 7u) == 0);
    if (vec && p.V <= kCeMaxChunks * kCeThreads * 8)      k_ce_rows<QUANT, kCeThreads><<<rows, kCeThreads, 0, st>>>(p);
    else if (vec && p.V <= kCeMaxChunks * kCeWide * 8)    k_ce_rows<QUANT, kCeWide><<<rows, kCeWide, 0, st>>>(p);
    else if (vec)                                         k_ce_rows_stream<QUANT><<<rows, kCeThreads, 0, st>>>(p);
    else                                             k_ce_rows_generic<QUANT><<<rows, kCeThreads, 0, st>>>(p);
    return launch_status();
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_cross_entropy_count_valid(const int32_t* d_labels, int n, int* d_n_valid, cf_stream_t stream) {
    if (n < 0 || !d_n_valid || (n > 0 && !d_labels)) return CF_ERR_INVALID_ARG;
    if (n == 0) return CF_OK;
    const unsigned blocks = min(ceil_div(n, kCeThreads), 256u);      // kernels/cross_entropy.cu:284-286
    k_count_valid<<<blocks, kCeThreads, 0, as_stream(stream)>>>(d_labels, n, d_n_valid);
    return launch_status();
}

int cf_cross_entropy_fwd_bwd_chunk(const uint16_t* d_logits, const int32_t* d_labels, float* d_loss_out, uint16_t* d_grad,
                                   int rows, int V, const int* d_n_valid, cf_stream_t stream) {
    if (rows < 0 || V < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || V == 0) return CF_OK;
    if (!d_logits || !d_labels || !d_loss_out || !d_grad || !d_n_valid) return CF_ERR_INVALID_ARG;
    CeArgs p{d_logits, d_labels, d_loss_out, d_grad, d_n_valid, nullptr, nullptr, nullptr, V};
    return launch_ce<false>(p, rows, as_stream(stream));
}

int cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(const uint16_t* d_logits, const int32_t* d_labels, float* d_loss_out,
                                              uint16_t* d_grad, void* d_grad8, const float* d_qscale, float* d_amax,
                                              int rows, int V, const int* d_n_valid, cf_stream_t stream) {
    if (rows < 0 || V < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || V == 0) return CF_OK;
    if (!d_logits || !d_labels || !d_loss_out || !d_grad || !d_n_valid || !d_grad8 || !d_qscale || !d_amax) return CF_ERR_INVALID_ARG;
    CeArgs p{d_logits, d_labels, d_loss_out, d_grad, d_n_valid, static_cast<uint8_t*>(d_grad8), d_qscale, d_amax, V};
    return launch_ce<true>(p, rows, as_stream(stream));
}

}  // extern "C"
