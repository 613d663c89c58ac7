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

// Large tensors: silu(g) in fp32 depends on the 16 bits of g only, and the reproducible exponential behind it costs
// about 40 vector instructions, which is what the plain kernels wait for.  A workgroup that stays on its CU builds a
// table of g * sigmoid(g) (and of the derivative, for the backward) for every bf16 g with 2^-25 <= |g| < 128 with the
// same expressions, 4096 magnitudes x 2 signs, and looks each element up; the few values outside (zeros, tiny, huge,
// non-finite) are evaluated directly.  Same bits either way.
constexpr int kLutThreads = 1024;
constexpr uint32_t kSiluLo = 0x3300u, kSiluSpan = 0x1000u;      // bf16 magnitudes 2^-25 .. 128

__device__ __forceinline__ float silu_direct(float g) { return g * stable_sigmoid(g); }
__device__ __forceinline__ float dsilu_direct(float g) {
    const float sg = stable_sigmoid(g);
    return sg * (1.0f + g * (1.0f - sg));
}
__device__ __forceinline__ uint32_t silu_slot(uint32_t b16) { return (b16 & 0x7fffu) - kSiluLo; }      // < kSiluSpan: in the table

template <bool BWD>
__device__ __forceinline__ void build_silu_lut(float* lut) {
    for (uint32_t i = threadIdx.x; i < 2 * kSiluSpan; i += kLutThreads) {
        const float g = bf16_to_f32(static_cast<uint16_t>((i >= kSiluSpan ? 0x8000u : 0u) | (kSiluLo + (i & (kSiluSpan - 1)))));
        lut[i] = silu_direct(g);
        if constexpr (BWD) lut[2 * kSiluSpan + i] = dsilu_direct(g);
    }
    __syncthreads();
}

__global__ __launch_bounds__(kLutThreads) void k_swiglu_lut(const uint4* __restrict__ gate, const uint4* __restrict__ up,
                                                            uint4* __restrict__ out, size_t nvec) {
    __shared__ float lut[2 * kSiluSpan];
    build_silu_lut<false>(lut);
    auto silu = [&](uint32_t b16) {
        const uint32_t slot = silu_slot(b16);
        return slot < kSiluSpan ? lut[slot + (b16 >> 15) * kSiluSpan] : silu_direct(bf16_to_f32(static_cast<uint16_t>(b16)));
    };
    auto one = [&](uint32_t g, uint32_t u) { return pack_bf16x2_hw(silu(g & 0xffffu) * bf16_lo(u), silu(g >> 16) * bf16_hi(u)); };
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const uint4 g = gate[i], u = up[i];
        store_stream16(out + i, make_uint4(one(g.x, u.x), one(g.y, u.y), one(g.z, u.z), one(g.w, u.w)));
    }
}

__global__ __launch_bounds__(kLutThreads) void k_swiglu_bwd_lut(const uint4* __restrict__ grad, const uint4* __restrict__ gate,
                                                                const uint4* __restrict__ up, uint4* __restrict__ dgate,
                                                                uint4* __restrict__ dup, size_t nvec) {
    __shared__ float lut[4 * kSiluSpan];
    build_silu_lut<true>(lut);
    auto one = [&](uint32_t d, uint32_t g, uint32_t u, uint32_t& og, uint32_t& ou) {
        float a[2], b[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t b16 = h ? g >> 16 : g & 0xffffu;
            const float dv = h ? bf16_hi(d) : bf16_lo(d), uv = h ? bf16_hi(u) : bf16_lo(u);
            const uint32_t slot = silu_slot(b16);
            float s, ds;
            if (slot < kSiluSpan) {
                s = lut[slot + (b16 >> 15) * kSiluSpan];
                ds = lut[2 * kSiluSpan + slot + (b16 >> 15) * kSiluSpan];
            } else {
                const float gv = bf16_to_f32(static_cast<uint16_t>(b16));
                s = silu_direct(gv);
                ds = dsilu_direct(gv);
            }
            a[h] = (dv * uv) * ds;
            b[h] = dv * s;
        }
        og = pack_bf16x2_hw(a[0], a[1]);
        ou = pack_bf16x2_hw(b[0], b[1]);
    };
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const uint4 d = grad[i], g = gate[i], u = up[i];
        uint4 og, ou;
        one(d.x, g.x, u.x, og.x, ou.x); one(d.y, g.y, u.y, og.y, ou.y); one(d.z, g.z, u.z, og.z, ou.z); one(d.w, g.w, u.w, og.w, ou.w);
        store_stream16(dgate + i, og);
        store_stream16(dup + i, ou);
    }
}

constexpr size_t kLutMinVecs = 32768;      // 256 Ki elements: from here on the tables pay for themselves

inline int lut_grid() {
    static int cus = [] {
        int dev = 0, c = 0;
        return (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && c > 0) ? c : 256;
    }();
    return cus;
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
// in LDS, the first wavefront walks each tile with one column per lane, four rows per (transposing) LDS read.
constexpr int kCsCols = 64, kCsRows = 128, kCsChunks = kCsRows * kCsCols / 8 / kThreads;   // 4 chunks per thread and tile

// FAST: 16-byte aligned rows and cols % 8 == 0.  The fetches are buffer loads (a descriptor with the tensor's size;
// rows past the end and chunks past the last column read as zeros), issued unconditionally four tiles ahead of the
// sum: with loads under branches the compiler cannot count the loads in flight and waits for all of them before the
// first LDS store, which leaves one tile in flight per workgroup.  Otherwise: element-wise guarded loads, two tiles.
template <bool FAST>
__global__ __launch_bounds__(kThreads) void k_col_sum(const uint16_t* __restrict__ in, float* __restrict__ out_accum,
                                                      int rows, int cols, int row_stride, int base) {
    __shared__ __attribute__((aligned(16))) uint16_t tile[2][kCsRows][kCsCols];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c0 = blockIdx.x * kCsCols;
    const int chunk = tid & 7, crow = tid >> 3;            // this thread's 8 columns, its row within each group of 32
    const int ccol = c0 + chunk * 8;
    const uint16_t* src = in + base + ccol;
    const int ntiles = (rows + kCsRows - 1) / kCsRows;
    constexpr int DEPTH = FAST ? 4 : 2;

    // FAST: the descriptor starts at this workgroup's first column and ends with the last row's last column
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const uint32_t span = static_cast<uint32_t>(max(rows - 1, 0)) * static_cast<uint32_t>(row_stride) * 2u +
                          static_cast<uint32_t>(max(min(kCsCols, cols - c0), 0)) * 2u;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(in + base + c0), 0,
                                                                        static_cast<int>(rows > 0 ? span : 0u), 0x00020000);
    const uint32_t lane_off = ccol < cols ? static_cast<uint32_t>(crow) * static_cast<uint32_t>(row_stride) * 2u + chunk * 16u : 0x80000000u;

    auto fetch = [&](int t, uint4 (&r)[kCsChunks]) {
#pragma unroll
        for (int i = 0; i < kCsChunks; ++i) {
            if constexpr (FAST) {
                // the row group's offset is uniform: it goes into the scalar part of the address
                const uint32_t group = static_cast<uint32_t>(t * kCsRows + i * 32) * static_cast<uint32_t>(row_stride) * 2u;
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<int>(lane_off + group), 0, 0);
                r[i] = make_uint4(v.x, v.y, v.z, v.w);
            } else {
                const int row = t * kCsRows + i * 32 + crow;
                r[i] = make_uint4(0, 0, 0, 0);
                if (row >= rows || ccol >= cols) continue;
                const uint16_t* p = src + static_cast<size_t>(row) * row_stride;
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
    float acc = 0.0f;
    // Rows past the end of the tensor are parked as zeros, and a running sum that started at +0 never is -0, so adding
    // them changes nothing: every tile is walked in full, and so are the tiles past the last one that round the loop
    // up to a multiple of DEPTH.  One transposing read hands a lane four consecutive rows of its column (per 16 lanes
    // a 4 x 16 block: source lane i supplies row i / 4, columns 4 (i % 4) .. +3 of the block's 16 columns; lane i
    // receives column i).
    typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4bf* lds_v4bf_ptr;
    const int i16 = lane & 15;
    auto sum_tile = [&](int buf) {
        if (wave != 0) return;
        const uint16_t* rd = &tile[buf][i16 >> 2][16 * (lane >> 4) + 4 * (i16 & 3)];
        // the next 32 rows are requested before the current 32 are added: an LDS round trip per read would otherwise
        // sit in the middle of the chain of dependent additions
        constexpr int B = 8;                                   // reads per batch
        v4bf cur[B], nxt[B];
#pragma unroll
        for (int j = 0; j < B; ++j) cur[j] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4bf_ptr)(rd + 4 * j * kCsCols));
#pragma unroll
        for (int r0 = 0; r0 < kCsRows; r0 += 4 * B) {
            if (r0 + 4 * B < kCsRows) {
#pragma unroll
                for (int j = 0; j < B; ++j)
                    nxt[j] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4bf_ptr)(rd + (r0 + 4 * B + 4 * j) * kCsCols));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < B; ++j) {
                acc += static_cast<float>(cur[j][0]);
                acc += static_cast<float>(cur[j][1]);
                acc += static_cast<float>(cur[j][2]);
                acc += static_cast<float>(cur[j][3]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < B; ++j) cur[j] = nxt[j];
        }
    };

    // DEPTH register sets hold the tiles t .. t + DEPTH - 1; one barrier per tile: the LDS buffer written at a step
    // was last read two steps earlier, and the summing wavefront has passed the barrier in between only after that.
    uint4 r[DEPTH][kCsChunks];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) fetch(d, r[d]);
    for (int t = 0; t < ntiles; t += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            park(d & 1, r[d]);
            fetch(t + d + DEPTH, r[d]);
            __syncthreads();
            sum_tile(d & 1);
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

// A measuring stick, not part of the hot path: the memory traffic of a per-token quantize (32 bytes read, 16 written
// per lane and step, one wavefront per row, the same streaming stores) with next to no arithmetic, so that what such
// a kernel could reach on this part can be read beside what the quantize kernels do reach.
__global__ __launch_bounds__(kThreads) void k_stream_2r1w(const uint4* __restrict__ src, uint4* __restrict__ dst, int rows, int steps) {
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const uint4* s = src + static_cast<size_t>(row) * steps * 128;
    uint4* d = dst + static_cast<size_t>(row) * steps * 64;
    for (int i = 0; i < steps; ++i) {
        const uint4 a = s[(i * 64 + lane) * 2], b = s[(i * 64 + lane) * 2 + 1];
        store_stream16(d + i * 64 + lane, make_uint4(a.x ^ b.x, a.y ^ b.y, a.z ^ b.z, a.w ^ b.w));
    }
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
    if (vec && static_cast<size_t>(n) / 8 >= kLutMinVecs) {
        const size_t nvec = static_cast<size_t>(n) / 8;
        hipStream_t st = as_stream(stream);
        k_swiglu_lut<<<lut_grid(), kLutThreads, 0, st>>>(reinterpret_cast<const uint4*>(d_gate), reinterpret_cast<const uint4*>(d_up),
                                                        reinterpret_cast<uint4*>(d_out), nvec);
        const int rest = n - static_cast<int>(nvec * 8);
        if (rest > 0) k_swiglu<<<1, kThreads, 0, st>>>(d_gate + nvec * 8, d_up + nvec * 8, d_out + nvec * 8, rest, 0);
        return launch_status();
    }
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
    if (vec && static_cast<size_t>(n) / 8 >= kLutMinVecs) {
        const size_t nvec = static_cast<size_t>(n) / 8;
        hipStream_t st = as_stream(stream);
        k_swiglu_bwd_lut<<<lut_grid(), kLutThreads, 0, st>>>(reinterpret_cast<const uint4*>(d_grad_out), reinterpret_cast<const uint4*>(d_gate),
                                                            reinterpret_cast<const uint4*>(d_up), reinterpret_cast<uint4*>(d_grad_gate),
                                                            reinterpret_cast<uint4*>(d_grad_up), nvec);
        const int rest = n - static_cast<int>(nvec * 8);
        if (rest > 0)
            k_swiglu_bwd<<<1, kThreads, 0, st>>>(d_grad_out + nvec * 8, d_gate + nvec * 8, d_up + nvec * 8, d_grad_gate + nvec * 8,
                                                 d_grad_up + nvec * 8, rest, 0);
        return launch_status();
    }
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
    // 16-byte chunks: every chunk of every row must be aligned and whole, and offsets must fit 31 bits
    const bool fast = aligned16(d_in) && row_stride % 8 == 0 && base % 8 == 0 && cols % 8 == 0 && row_stride >= cols &&
                      static_cast<size_t>(rows) * row_stride < (1ull << 30);
    const dim3 grid(ceil_div(cols, kCsCols));
    if (fast) k_col_sum<true><<<grid, kThreads, 0, as_stream(stream)>>>(d_in, d_out_accum, rows, cols, row_stride, base);
    else      k_col_sum<false><<<grid, kThreads, 0, as_stream(stream)>>>(d_in, d_out_accum, rows, cols, row_stride, base);
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

int cf_hbm_stream_probe_2r1w(const void* d_src, void* d_dst, int rows, int row_bytes_out, cf_stream_t stream) {
    if (rows < 0 || row_bytes_out < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || row_bytes_out == 0) return CF_OK;
    if (!d_src || !d_dst) return CF_ERR_INVALID_ARG;
    if (row_bytes_out % 1024 != 0 || !aligned16(d_src) || !aligned16(d_dst)) return CF_ERR_UNSUPPORTED;
    k_stream_2r1w<<<ceil_div(rows, kThreads / 64), kThreads, 0, as_stream(stream)>>>(static_cast<const uint4*>(d_src),
                                                                                     static_cast<uint4*>(d_dst), rows, row_bytes_out / 1024);
    return launch_status();
}

}  // extern "C"
