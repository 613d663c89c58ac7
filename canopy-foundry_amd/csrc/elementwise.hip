// Stand-alone forms of the bf16 epilogue ops (SiLU-gate forward and backward, strided bias add and its
// gradient, the column sum).  The GEMM fuses the forward arithmetic into its epilogue; these exist because
// the reference exposes them as separate entry points.
#include "common.hpp"

namespace cf {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ uint16_t swiglu1(uint16_t g, uint16_t u) {
    const float gv = bf16_to_f32(g), uv = bf16_to_f32(u);
    return f32_to_bf16((gv * stable_sigmoid(gv)) * uv);
}
__device__ __forceinline__ uint32_t swiglu2(uint32_t g, uint32_t u) {
    const float g0 = bf16_lo(g), g1 = bf16_hi(g);
    return pack_bf16x2_hw((g0 * stable_sigmoid(g0)) * bf16_lo(u), (g1 * stable_sigmoid(g1)) * bf16_hi(u));
}

__global__ __launch_bounds__(kThreads) void k_swiglu(const uint16_t* __restrict__ gate,
                                                     const uint16_t* __restrict__ up,
                                                     uint16_t* __restrict__ out, int n, int vec) {
    const int tid = blockIdx.x * blockDim.x + threadIdx.x;
    const int stride = gridDim.x * blockDim.x;
    int done = 0;
    if (vec) {
        const int nvec = n / 8;
        for (int i = tid; i < nvec; i += stride) {
            const uint4 g = reinterpret_cast<const uint4*>(gate)[i];
            const uint4 u = reinterpret_cast<const uint4*>(up)[i];
            uint4 o;
            o.x = swiglu2(g.x, u.x); o.y = swiglu2(g.y, u.y); o.z = swiglu2(g.z, u.z); o.w = swiglu2(g.w, u.w);
            store_stream16(reinterpret_cast<uint4*>(out) + i, o);
        }
        done = nvec * 8;
    }
    for (int i = done + tid; i < n; i += stride) out[i] = swiglu1(gate[i], up[i]);
}

// swiglu_backward (kernels/activations.cu:42-58 of the reference): one sigmoid serves silu and its derivative;
// the products are taken in the reference's order.
__device__ __forceinline__ void swiglu_bwd1(float d, float g, float u, float& dg, float& du) {
    const float sg = stable_sigmoid(g);
    const float dsilu = sg * (1.0f + g * (1.0f - sg));
    dg = (d * u) * dsilu;
    du = d * (g * sg);
}
__device__ __forceinline__ void swiglu_bwd2(uint32_t d, uint32_t g, uint32_t u, uint32_t& dg, uint32_t& du) {
    float a0, a1, b0, b1;
    swiglu_bwd1(bf16_lo(d), bf16_lo(g), bf16_lo(u), a0, b0);
    swiglu_bwd1(bf16_hi(d), bf16_hi(g), bf16_hi(u), a1, b1);
    dg = pack_bf16x2_hw(a0, a1);
    du = pack_bf16x2_hw(b0, b1);
}

// 10 bytes per element (three bf16 read, two written): 16-byte accesses when all five pointers allow it
__global__ __launch_bounds__(kThreads) void k_swiglu_bwd(const uint16_t* __restrict__ grad, const uint16_t* __restrict__ gate,
                                                         const uint16_t* __restrict__ up, uint16_t* __restrict__ dgate,
                                                         uint16_t* __restrict__ dup, int n, int vec) {
    const int tid = blockIdx.x * blockDim.x + threadIdx.x;
    const int stride = gridDim.x * blockDim.x;
    int done = 0;
    if (vec) {
        const int nvec = n / 8;
        for (int i = tid; i < nvec; i += stride) {
            const uint4 d = reinterpret_cast<const uint4*>(grad)[i];
            const uint4 g = reinterpret_cast<const uint4*>(gate)[i];
            const uint4 u = reinterpret_cast<const uint4*>(up)[i];
            uint4 og, ou;
            swiglu_bwd2(d.x, g.x, u.x, og.x, ou.x); swiglu_bwd2(d.y, g.y, u.y, og.y, ou.y);
            swiglu_bwd2(d.z, g.z, u.z, og.z, ou.z); swiglu_bwd2(d.w, g.w, u.w, og.w, ou.w);
            store_stream16(reinterpret_cast<uint4*>(dgate) + i, og);
            store_stream16(reinterpret_cast<uint4*>(dup) + i, ou);
        }
        done = nvec * 8;
    }
    for (int i = done + tid; i < n; i += stride) {
        float a, b;
        swiglu_bwd1(bf16_to_f32(grad[i]), bf16_to_f32(gate[i]), bf16_to_f32(up[i]), a, b);
        dgate[i] = f32_to_bf16(a);
        dup[i] = f32_to_bf16(b);
    }
}

// Column sum over rows in ascending row order, one fp32 chain per column from zero (the reference's order, so the
// sum has the reference's bits).  The chain is serial, the memory traffic need not be: a workgroup owns 64
// columns, all four wavefronts fetch tiles of 128 rows (16-byte chunks, two tiles ahead of the sum) and park them
// in LDS, the first wavefront walks each tile row by row with one column per lane.
constexpr int kCsCols = 64, kCsRows = 128, kCsChunks = kCsRows * kCsCols / 8 / kThreads;   // 4 chunks per thread and tile

__global__ __launch_bounds__(kThreads) void k_col_sum(const uint16_t* __restrict__ in, float* __restrict__ out_accum,
                                                      int rows, int cols, int row_stride, int base, int vec) {
    __shared__ __attribute__((aligned(16))) uint16_t tile[2][kCsRows][kCsCols];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c0 = blockIdx.x * kCsCols;
    const int chunk = tid & 7, crow = tid >> 3;            // this thread's 8 columns, its row within each group of 32
    const int ccol = c0 + chunk * 8;
    const uint16_t* src = in + base + ccol;
    const int ntiles = (rows + kCsRows - 1) / kCsRows;

    auto fetch = [&](int t, uint4 (&r)[kCsChunks]) {
#pragma unroll
        for (int i = 0; i < kCsChunks; ++i) {
            const int row = t * kCsRows + i * 32 + crow;
            r[i] = make_uint4(0, 0, 0, 0);
            if (row >= rows || ccol >= cols) continue;
            const uint16_t* p = src + static_cast<size_t>(row) * row_stride;
            if (vec && ccol + 8 <= cols) {
                r[i] = *reinterpret_cast<const uint4*>(p);
            } else {
                uint16_t e[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) e[q] = ccol + q < cols ? p[q] : static_cast<uint16_t>(0);
                r[i] = make_uint4(e[0] | (uint32_t)e[1] << 16, e[2] | (uint32_t)e[3] << 16, e[4] | (uint32_t)e[5] << 16,
                                  e[6] | (uint32_t)e[7] << 16);
            }
        }
    };
    auto park = [&](int buf, const uint4 (&r)[kCsChunks]) {
#pragma unroll
        for (int i = 0; i < kCsChunks; ++i) *reinterpret_cast<uint4*>(&tile[buf][i * 32 + crow][chunk * 8]) = r[i];
    };

    uint4 ra[kCsChunks], rb[kCsChunks];      // tiles t+1 and t+2 while tile t is summed
    float acc = 0.0f;
    fetch(0, ra);
    if (ntiles > 1) fetch(1, rb);
    for (int t = 0; t < ntiles; ++t) {
        // tile t is in ra for even t, in rb for odd t
        if (t & 1) park(1, rb); else park(0, ra);
        if (t + 2 < ntiles) { if (t & 1) fetch(t + 2, rb); else fetch(t + 2, ra); }
        // One barrier per tile: the buffer written here was last read two tiles ago, and the first wavefront has
        // passed the barrier in between only after finishing that read.
        __syncthreads();
        if (wave == 0) {
            const int nr = min(kCsRows, rows - t * kCsRows);
            if (nr == kCsRows) {
#pragma unroll 16
                for (int r = 0; r < kCsRows; ++r) acc += bf16_to_f32(tile[t & 1][r][lane]);
            } else {
                for (int r = 0; r < nr; ++r) acc += bf16_to_f32(tile[t & 1][r][lane]);
            }
        }
    }
    if (wave == 0 && c0 + lane < cols) out_accum[c0 + lane] += acc;
}

__global__ __launch_bounds__(kThreads) void k_bias_add(uint16_t* __restrict__ inout,
                                                       const uint16_t* __restrict__ bias, int cols,
                                                       int row_stride, int base) {
    uint16_t* row = inout + static_cast<size_t>(blockIdx.x) * row_stride + base;
    for (int c = threadIdx.x; c < cols; c += blockDim.x)
        row[c] = f32_to_bf16(bf16_to_f32(row[c]) + bf16_to_f32(bias[c]));
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_swiglu_forward(const uint16_t* d_gate, const uint16_t* d_up, uint16_t* d_out, int n, cf_stream_t stream) {
    if (n < 0) return CF_ERR_INVALID_ARG;
    if (n == 0) return CF_OK;
    if (!d_gate || !d_up || !d_out) return CF_ERR_INVALID_ARG;
    const int vec = aligned16(d_gate) && aligned16(d_up) && aligned16(d_out);
    const size_t items = vec ? (static_cast<size_t>(n) + 7) / 8 : static_cast<size_t>(n);
    size_t blocks = (items + kThreads - 1) / kThreads;
    if (blocks > 8192) blocks = 8192;
    k_swiglu<<<static_cast<unsigned>(blocks), kThreads, 0, as_stream(stream)>>>(d_gate, d_up, d_out, n, vec);
    return launch_status();
}

int cf_swiglu_backward(const uint16_t* d_grad_out, const uint16_t* d_gate, const uint16_t* d_up, uint16_t* d_grad_gate,
                       uint16_t* d_grad_up, int n, cf_stream_t stream) {
    if (n < 0) return CF_ERR_INVALID_ARG;
    if (n == 0) return CF_OK;
    if (!d_grad_out || !d_gate || !d_up || !d_grad_gate || !d_grad_up) return CF_ERR_INVALID_ARG;
    const int vec = aligned16(d_grad_out) && aligned16(d_gate) && aligned16(d_up) && aligned16(d_grad_gate) && aligned16(d_grad_up);
    const size_t items = vec ? (static_cast<size_t>(n) + 7) / 8 : static_cast<size_t>(n);
    size_t blocks = (items + kThreads - 1) / kThreads;
    if (blocks > 8192) blocks = 8192;
    k_swiglu_bwd<<<static_cast<unsigned>(blocks), kThreads, 0, as_stream(stream)>>>(d_grad_out, d_gate, d_up, d_grad_gate,
                                                                                    d_grad_up, n, vec);
    return launch_status();
}

int cf_col_sum_strided_bf16(const uint16_t* d_in, float* d_out_accum, int rows, int cols, int row_stride, int base,
                            cf_stream_t stream) {
    if (rows < 0 || cols < 0 || base < 0) return CF_ERR_INVALID_ARG;
    if (cols == 0) return CF_OK;
    if (!d_out_accum || (rows > 0 && !d_in)) return CF_ERR_INVALID_ARG;
    // 16-byte chunks: every chunk of every row must be aligned
    const int vec = aligned16(d_in) && row_stride % 8 == 0 && base % 8 == 0;
    k_col_sum<<<ceil_div(cols, kCsCols), kThreads, 0, as_stream(stream)>>>(d_in, d_out_accum, rows, cols, row_stride, base, vec);
    return launch_status();
}

int cf_bias_add_strided_bf16(uint16_t* d_inout, const uint16_t* d_bias, int rows, int cols, int row_stride,
                             int base, cf_stream_t stream) {
    if (rows < 0 || cols < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return CF_OK;
    if (!d_inout || !d_bias) return CF_ERR_INVALID_ARG;
    k_bias_add<<<rows, kThreads, 0, as_stream(stream)>>>(d_inout, d_bias, cols, row_stride, base);
    return launch_status();
}

const char* cf_version(void) { return "canopy-foundry_amd fp8 hot path, gfx950"; }

}  // extern "C"
