// Stand-alone forms of the bf16 epilogue ops (SiLU-gate, strided bias add).
// The GEMM fuses the same arithmetic into its epilogue; these exist because the
// reference exposes them as separate entry points.
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
