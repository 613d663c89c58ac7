// Custom kernels of the MoE expert-bank backward that reuses the forward's routes (saved counts, offsets and
// per-expert row lists): exact-erf GELU forward and backward, and the two uses of the upstream gradient per
// selected (row, expert) pair,
//     d_route_weight[row, e] = dot(d_mixed[row], expert_out[slot])
//     d_expert_out[slot]     = bf16(route_weight[row, e] * d_mixed[row]),
// one launch per expert in the reference.  The grouped form here walks every expert's list in one launch and
// fuses the two: a row of d_mixed and a row of expert_out are read once, the gradient row overwrites the
// expert_out row it was read from.
//
// The dot is bit-reproducible.  Products of two bf16 values are exact in fp32, so only the summation tree
// matters, and it is the reference's: T = min(H, 256) threads, thread t sums h = t, t + T, ... in order, then a
// halving tree over the T partials (strides T/2 .. 1).  With H % 256 == 0 half a wavefront takes a row: lane l
// of the half holds elements 256 s + 8 l .. + 7 of stripe s (one 16-byte load), that is one link of the chains of
// threads 8 l .. 8 l + 7; the tree's strides 128 .. 8 are exchanges across lanes (xor 16 .. 1), 4, 2, 1 in-lane.
// Any other H takes a workgroup of T threads per row and the tree through LDS.
#include "common.hpp"
#include <mutex>

namespace cf {
namespace {

constexpr int kThreads = 256;

struct RouteGradArgs {
    const uint16_t* a_full;     // [rows, H]: the upstream gradient, indexed by token row
    const uint16_t* b;          // [slots, H]: dot operand, indexed by slot (DOT)
    uint16_t* dst;              // [slots, H]: route-weighted copy of a_full's rows (SCALE); may be b
    float* out;                 // dot results at out[row * out_stride + column]
    const float* rw;            // [rows, E] route weights (SCALE)
    const int* counts;          // grouped: per-expert list lengths; null: one list of n_single rows
    const int* offsets;         // grouped: first slot of each expert
    const int* row_indices;     // grouped: [E, rows] lists; otherwise the one list
    int n_single, expert_idx, out_col;
    int rows, E, H, out_stride;
};

__device__ __forceinline__ float bf16_elem(const uint4& v, int i) {
    const uint32_t w = (i < 2) ? v.x : (i < 4) ? v.y : (i < 6) ? v.z : v.w;
    return (i & 1) ? bf16_hi(w) : bf16_lo(w);
}
__device__ __forceinline__ uint32_t scale2_bf16(uint32_t pair, float w) {
    return pack_bf16x2(w * bf16_lo(pair), w * bf16_hi(pair));
}

// H % 256 == 0, 16-byte aligned rows.  grid (x, experts or 1); a workgroup takes eight slots per step.
template <bool DOT, bool SCALE>
__global__ __launch_bounds__(kThreads) void k_route_grad_half_wave(const RouteGradArgs p) {
    const int e = p.counts ? static_cast<int>(blockIdx.y) : p.expert_idx;
    const int n = p.counts ? p.counts[e] : p.n_single;
    const int base = p.counts ? p.offsets[e] : 0;
    const int* list = p.counts ? p.row_indices + static_cast<size_t>(e) * p.rows : p.row_indices;
    const int col = p.counts ? e : p.out_col;
    const int half = threadIdx.x >> 5, l = threadIdx.x & 31;
    const int stripes = p.H >> 8;
    for (int i = blockIdx.x * 8 + half; i < n; i += gridDim.x * 8) {
        const int row = list[i];
        const size_t slot = static_cast<size_t>(base) + i;
        const uint4* a = reinterpret_cast<const uint4*>(p.a_full + static_cast<size_t>(row) * p.H) + l;
        const uint4* b = DOT ? reinterpret_cast<const uint4*>(p.b + slot * p.H) + l : nullptr;
        uint4* d = SCALE ? reinterpret_cast<uint4*>(p.dst + slot * p.H) + l : nullptr;
        const float w = SCALE ? p.rw[static_cast<size_t>(row) * p.E + e] : 0.0f;
        float part[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 4
        for (int s = 0; s < stripes; ++s) {
            const uint4 av = a[s * 32];
            if constexpr (DOT) {
                const uint4 bv = b[s * 32];
#pragma unroll
                for (int j = 0; j < 8; ++j) part[j] = __builtin_fmaf(bf16_elem(av, j), bf16_elem(bv, j), part[j]);
            }
            if constexpr (SCALE)
                store_stream16(d + s * 32, make_uint4(scale2_bf16(av.x, w), scale2_bf16(av.y, w), scale2_bf16(av.z, w), scale2_bf16(av.w, w)));
        }
        if constexpr (DOT) {
            // strides 128, 64, 32, 16, 8 of the halving tree
#pragma unroll
            for (int off = 16; off > 0; off >>= 1)
#pragma unroll
                for (int j = 0; j < 8; ++j) part[j] += __shfl_xor(part[j], off, kWave);
            // strides 4, 2, 1
            const float q0 = part[0] + part[4], q1 = part[1] + part[5], q2 = part[2] + part[6], q3 = part[3] + part[7];
            const float r0 = q0 + q2, r1 = q1 + q3;
            if (l == 0) p.out[static_cast<size_t>(row) * p.out_stride + col] = r0 + r1;
        }
    }
}

// Any H: one workgroup of T = min(H, 256) threads per slot, the reference's tree through LDS.
template <bool DOT, bool SCALE>
__global__ void k_route_grad_block(const RouteGradArgs p) {
    __shared__ float sh[256];
    const int e = p.counts ? static_cast<int>(blockIdx.y) : p.expert_idx;
    const int n = p.counts ? p.counts[e] : p.n_single;
    const int base = p.counts ? p.offsets[e] : 0;
    const int* list = p.counts ? p.row_indices + static_cast<size_t>(e) * p.rows : p.row_indices;
    const int col = p.counts ? e : p.out_col;
    const int t = threadIdx.x, T = blockDim.x;
    for (int i = blockIdx.x; i < n; i += gridDim.x) {
        const int row = list[i];
        const size_t slot = static_cast<size_t>(base) + i;
        const uint16_t* a = p.a_full + static_cast<size_t>(row) * p.H;
        const float w = SCALE ? p.rw[static_cast<size_t>(row) * p.E + e] : 0.0f;
        float sum = 0.0f;
        for (int h = t; h < p.H; h += T) {
            const float av = bf16_to_f32(a[h]);
            if constexpr (DOT) sum = __builtin_fmaf(av, bf16_to_f32(p.b[slot * p.H + h]), sum);
            if constexpr (SCALE) p.dst[slot * p.H + h] = f32_to_bf16(w * av);
        }
        if constexpr (DOT) {
            sh[t] = sum;
            __syncthreads();
            for (int stride = T / 2; stride > 0; stride >>= 1) {
                if (t < stride) sh[t] += sh[t + stride];
                __syncthreads();
            }
            if (t == 0) p.out[static_cast<size_t>(row) * p.out_stride + col] = sh[0];
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(kThreads) void k_fill_zero_f32(float* x, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        x[i] = 0.0f;
}

template <bool DOT, bool SCALE>
int launch_route_grad(const RouteGradArgs& p, int max_list, hipStream_t st) {
    const int experts = p.counts ? p.E : 1;
    const bool vec = p.H % 256 == 0 && aligned16(p.a_full) && (!DOT || aligned16(p.b)) && (!SCALE || aligned16(p.dst));
    if (vec) {
        // enough workgroups for the longest possible list without making empty experts expensive
        const unsigned gx = static_cast<unsigned>(min(ceil_div(static_cast<size_t>(max_list), 8), ceil_div(8192, static_cast<size_t>(experts))));
        k_route_grad_half_wave<DOT, SCALE><<<dim3(gx ? gx : 1, experts), kThreads, 0, st>>>(p);
    } else {
        const int T = p.H < 256 ? p.H : 256;
        const unsigned gx = static_cast<unsigned>(min(static_cast<size_t>(max_list), static_cast<size_t>(ceil_div(65536, static_cast<size_t>(experts)))));
        k_route_grad_block<DOT, SCALE><<<dim3(gx ? gx : 1, experts), T, 0, st>>>(p);
    }
    return launch_status();
}

// ---- GELU ----------------------------------------------------------------------------------------
// `cdf + x * pdf` is one fused multiply-add in the reference's build (default contraction)
__device__ __forceinline__ float gelu_deriv(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.7071067811865476f));
    const float pdf = 0.3989422804014327f * expf(-0.5f * x * x);
    return __builtin_fmaf(x, pdf, cdf);
}
__device__ __forceinline__ uint32_t gelu_bwd2(uint32_t pre, uint32_t g) {
    return pack_bf16x2(bf16_lo(g) * gelu_deriv(bf16_lo(pre)), bf16_hi(g) * gelu_deriv(bf16_hi(pre)));
}

template <bool BWD>
__global__ __launch_bounds__(kThreads) void k_gelu_vec(const uint4* __restrict__ x, const uint4* __restrict__ g,
                                                       uint4* __restrict__ out, size_t nvec) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const uint4 v = x[i];
        if constexpr (BWD) {
            const uint4 u = g[i];
            store_stream16(out + i, make_uint4(gelu_bwd2(v.x, u.x), gelu_bwd2(v.y, u.y), gelu_bwd2(v.z, u.z), gelu_bwd2(v.w, u.w)));
        } else {
            store_stream16(out + i, make_uint4(gelu2(v.x), gelu2(v.y), gelu2(v.z), gelu2(v.w)));
        }
    }
}
template <bool BWD>
__global__ __launch_bounds__(kThreads) void k_gelu_scalar(const uint16_t* __restrict__ x, const uint16_t* __restrict__ g,
                                                          uint16_t* __restrict__ out, size_t first, size_t n) {
    for (size_t i = first + static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const float v = bf16_to_f32(x[i]);
        out[i] = f32_to_bf16(BWD ? bf16_to_f32(g[i]) * gelu_deriv(v) : gelu_fwd(v));
    }
}

// The forward for large tensors: bf16(gelu(x)) depends on the 16 bits of x only, so a workgroup that stays on its CU
// builds the table of all 65536 results once (128 KiB of LDS) and looks every element up; erff costs about 40 vector
// instructions per element and is what the plain kernel waits for.  Same bits.
constexpr int kLutThreads = 1024;
__global__ __launch_bounds__(kLutThreads) void k_gelu_lut(const uint4* __restrict__ x, uint4* __restrict__ out, size_t nvec) {
    extern __shared__ uint16_t lut[];
    for (int i = threadIdx.x; i < 65536; i += kLutThreads) lut[i] = f32_to_bf16(gelu_fwd(bf16_to_f32(static_cast<uint16_t>(i))));
    __syncthreads();
    auto look2 = [&](uint32_t pair) { return static_cast<uint32_t>(lut[pair & 0xffffu]) | (static_cast<uint32_t>(lut[pair >> 16]) << 16); };
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const uint4 v = x[i];
        store_stream16(out + i, make_uint4(look2(v.x), look2(v.y), look2(v.z), look2(v.w)));
    }
}

// The backward for large tensors: the derivative in fp32 depends on the 16 bits of the pre-activation only; erff and
// expf are what the plain kernel waits for.  A workgroup that stays on its CU builds the table of the derivative for
// every bf16 pre-activation with 2^-25 <= |x| < 128 (4096 magnitudes x 2 signs, 32 KiB) with the same expression; the
// few values outside (zeros, tiny, huge, non-finite) are evaluated directly.  Same bits either way.
constexpr uint32_t kDerivLo = 0x3300u, kDerivSpan = 0x1000u;
__global__ __launch_bounds__(kLutThreads) void k_gelu_bwd_lut(const uint4* __restrict__ x, const uint4* __restrict__ g,
                                                              uint4* __restrict__ out, size_t nvec) {
    __shared__ float lut[2 * kDerivSpan];
    for (uint32_t i = threadIdx.x; i < 2 * kDerivSpan; i += kLutThreads)
        lut[i] = gelu_deriv(bf16_to_f32(static_cast<uint16_t>((i >= kDerivSpan ? 0x8000u : 0u) | (kDerivLo + (i & (kDerivSpan - 1))))));
    __syncthreads();
    auto deriv = [&](uint32_t b16) {
        const uint32_t slot = (b16 & 0x7fffu) - kDerivLo;
        return slot < kDerivSpan ? lut[slot + (b16 >> 15) * kDerivSpan] : gelu_deriv(bf16_to_f32(static_cast<uint16_t>(b16)));
    };
    auto one = [&](uint32_t pre, uint32_t gr) { return pack_bf16x2(bf16_lo(gr) * deriv(pre & 0xffffu), bf16_hi(gr) * deriv(pre >> 16)); };
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const uint4 v = x[i], u = g[i];
        store_stream16(out + i, make_uint4(one(v.x, u.x), one(v.y, u.y), one(v.z, u.z), one(v.w, u.w)));
    }
}

template <bool BWD>
int launch_gelu(const uint16_t* x, const uint16_t* g, uint16_t* out, size_t n, hipStream_t st) {
    const bool vec = aligned16(x) && aligned16(out) && (!BWD || aligned16(g));
    const size_t nvec = vec ? n / 8 : 0;
    if constexpr (BWD) {
        if (nvec >= (1u << 17)) {        // 1 Mi elements: from here on 256 small tables pay for themselves
            static int cus = [] {
                int dev = 0, c = 0;
                return (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && c > 0) ? c : 256;
            }();
            k_gelu_bwd_lut<<<cus, kLutThreads, 0, st>>>(reinterpret_cast<const uint4*>(x), reinterpret_cast<const uint4*>(g),
                                                       reinterpret_cast<uint4*>(out), nvec);
            if (nvec * 8 < n)
                k_gelu_scalar<BWD><<<static_cast<unsigned>(min(ceil_div(n - nvec * 8, kThreads), 65536u)), kThreads, 0, st>>>(x, g, out, nvec * 8, n);
            return launch_status();
        }
    }
    if constexpr (!BWD) {
        if (nvec >= (8u << 20)) {        // 64 Mi elements: enough to pay for one table per CU
            static std::once_flag once;
            static hipError_t err = hipSuccess;
            static int cus = 256;
            std::call_once(once, [] {
                err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gelu_lut), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
                int dev = 0, c = 0;
                if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && c > 0)
                    cus = c;
            });
            if (err != hipSuccess) return static_cast<int>(err);
            k_gelu_lut<<<cus, kLutThreads, 128 * 1024, st>>>(reinterpret_cast<const uint4*>(x), reinterpret_cast<uint4*>(out), nvec);
            if (nvec * 8 < n)
                k_gelu_scalar<BWD><<<static_cast<unsigned>(min(ceil_div(n - nvec * 8, kThreads), 65536u)), kThreads, 0, st>>>(x, g, out, nvec * 8, n);
            return launch_status();
        }
    }
    if (nvec)
        k_gelu_vec<BWD><<<static_cast<unsigned>(min(ceil_div(nvec, kThreads), 65536u)), kThreads, 0, st>>>(
            reinterpret_cast<const uint4*>(x), reinterpret_cast<const uint4*>(g), reinterpret_cast<uint4*>(out), nvec);
    if (nvec * 8 < n)
        k_gelu_scalar<BWD><<<static_cast<unsigned>(min(ceil_div(n - nvec * 8, kThreads), 65536u)), kThreads, 0, st>>>(x, g, out, nvec * 8, n);
    return launch_status();
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_gelu_forward_bf16(const uint16_t* d_x, uint16_t* d_out, size_t n, cf_stream_t stream) {
    if (n == 0) return CF_OK;
    if (!d_x || !d_out) return CF_ERR_INVALID_ARG;
    return launch_gelu<false>(d_x, nullptr, d_out, n, as_stream(stream));
}

int cf_gelu_backward_bf16(const uint16_t* d_pre, const uint16_t* d_grad_post, uint16_t* d_grad_pre, size_t n,
                          cf_stream_t stream) {
    if (n == 0) return CF_OK;
    if (!d_pre || !d_grad_post || !d_grad_pre) return CF_ERR_INVALID_ARG;
    return launch_gelu<true>(d_pre, d_grad_post, d_grad_pre, n, as_stream(stream));
}

int cf_moe_row_dot_selected_bf16(const uint16_t* d_a_full, const uint16_t* d_b_compact, float* d_out,
                                 const int* d_row_indices, int n_rows, int H, int out_stride, int out_col,
                                 cf_stream_t stream) {
    if (n_rows < 0 || H < 0 || out_stride < 0 || out_col < 0) return CF_ERR_INVALID_ARG;
    if (n_rows == 0) return CF_OK;
    if (H == 0 || !d_a_full || !d_b_compact || !d_out || !d_row_indices) return CF_ERR_INVALID_ARG;
    RouteGradArgs p{};
    p.a_full = d_a_full; p.b = d_b_compact; p.out = d_out; p.row_indices = d_row_indices;
    p.n_single = n_rows; p.out_col = out_col; p.H = H; p.out_stride = out_stride; p.E = 1;
    return launch_route_grad<true, false>(p, n_rows, as_stream(stream));
}

int cf_moe_gather_scale_rows_bf16(const uint16_t* d_src, uint16_t* d_dst, const float* d_route_weights,
                                  const int* d_row_indices, int n_rows, int expert_idx, int num_experts, int H,
                                  cf_stream_t stream) {
    if (n_rows < 0 || H < 0 || num_experts <= 0 || expert_idx < 0 || expert_idx >= num_experts) return CF_ERR_INVALID_ARG;
    if (n_rows == 0 || H == 0) return CF_OK;
    if (!d_src || !d_dst || !d_route_weights || !d_row_indices) return CF_ERR_INVALID_ARG;
    RouteGradArgs p{};
    p.a_full = d_src; p.dst = d_dst; p.rw = d_route_weights; p.row_indices = d_row_indices;
    p.n_single = n_rows; p.expert_idx = expert_idx; p.E = num_experts; p.H = H;
    return launch_route_grad<false, true>(p, n_rows, as_stream(stream));
}

int cf_moe_grouped_route_grad_bf16(const uint16_t* d_grad_mixed, uint16_t* d_expert_out, float* d_grad_route_weights,
                                   const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                   const int* d_row_indices, int rows, int num_experts, int H, cf_stream_t stream) {
    if (rows < 0 || num_experts < 0 || H < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0) return CF_OK;
    if (H == 0 || !d_grad_mixed || !d_expert_out || !d_grad_route_weights || !d_route_weights || !d_counts || !d_offsets ||
        !d_row_indices)
        return CF_ERR_INVALID_ARG;
    hipStream_t st = as_stream(stream);
    // unselected (row, expert) pairs carry no gradient (src/trainer.cu:7667-7670 clears the buffer the same way)
    const size_t cells = static_cast<size_t>(rows) * num_experts;
    k_fill_zero_f32<<<static_cast<unsigned>(min(ceil_div(cells, kThreads), 4096u)), kThreads, 0, st>>>(d_grad_route_weights, cells);
    RouteGradArgs p{};
    p.a_full = d_grad_mixed; p.b = d_expert_out; p.dst = d_expert_out; p.out = d_grad_route_weights; p.rw = d_route_weights;
    p.counts = d_counts; p.offsets = d_offsets; p.row_indices = d_row_indices;
    p.rows = rows; p.E = num_experts; p.H = H; p.out_stride = num_experts;
    return launch_route_grad<true, true>(p, rows, st);
}

}  // extern "C"
