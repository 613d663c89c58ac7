// Transposing kernels for gfx950: bf16 -> E4M3 quantize with transposed output,
// the dual (straight + transposed) quantize, and the plain byte transpose that
// feeds the weight-gradient GEMM.
//
// Fast path (both extents multiples of 128, 16-byte aligned): a workgroup owns a
// 128 x 128 tile, a lane owns an 8 x 8 sub-block, transposes it in registers
// with v_perm_b32 (two 4x4 byte transposes per row group), stores 8-byte columns
// into LDS and the tile leaves as 128-byte row segments.  Other shapes take a
// 64 x 64 scalar tile.
#include "common.hpp"

namespace cf {
namespace {

constexpr int kThreads = 256;
constexpr int kTile = 128;
// LDS tile: [column][128 bytes of rows], no padding.  How this part serves LDS accesses decides the layout:
//  * an 8-byte store goes out for lanes 0-15 together with lanes 32-47 (and 16-31 with 48-63), and those 32 lanes
//    must hit 32 different 8-byte slots of a 256-byte line;
//  * a 16-byte load goes out for the lanes of 8-lane group G together with group G ^ 3, 16 different 16-byte slots.
// A lane stores 8 rows of one column per instruction.  Lanes 0-15 and 32-47 hold the two halves of one 16-byte chunk
// of rows (the row-block numbering below pairs them), sixteen neighbouring column blocks; odd column blocks store
// their columns in swapped pairs so that both 128-byte halves of a line are in use, and the 16-byte chunks of a
// column's row are xor-swizzled by column / 16.  The loads read whole 128-byte rows, and rows G and G ^ 3 differ in
// parity, i.e. sit in different halves.
constexpr int kPitch = kTile;

// rows r0..r3 hold bytes n0..n3; returns columns: c[j] = {r0.bj, r1.bj, r2.bj, r3.bj}
__device__ __forceinline__ void transpose4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t c[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    const uint32_t u0 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    const uint32_t u1 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c[0] = __builtin_amdgcn_perm(u0, t0, 0x05040100u);
    c[1] = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
    c[2] = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
    c[3] = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
}

// 8 consecutive source elements of one row -> 8 bytes
template <bool QUANT>
__device__ __forceinline__ uint2 load_row8(const void* src, size_t elem_index, float s) {
    if constexpr (QUANT) {
        const uint4 v = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(src) + elem_index);
        uint2 o;
        o.x = cvt4_fp8<false>(bf16_lo(v.x) * s, bf16_hi(v.x) * s, bf16_lo(v.y) * s, bf16_hi(v.y) * s);
        o.y = cvt4_fp8<false>(bf16_lo(v.z) * s, bf16_hi(v.z) * s, bf16_lo(v.w) * s, bf16_hi(v.w) * s);
        return o;
    } else {
        return *reinterpret_cast<const uint2*>(static_cast<const uint8_t*>(src) + elem_index);
    }
}

// in[R,C] (bf16 when QUANT, bytes otherwise) -> outT[C,R] bytes, and straight[R,C] when DUAL.
template <bool QUANT, bool DUAL>
__global__ __launch_bounds__(kThreads) void k_transpose_tiled(const void* __restrict__ in,
                                                              uint8_t* __restrict__ straight,
                                                              uint8_t* __restrict__ outT,
                                                              const float* __restrict__ scale, int R, int C) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTile * kPitch];   // [c][r]
    const int r0 = blockIdx.y * kTile, c0 = blockIdx.x * kTile;
    // lane = 16 * (row block within the wavefront) + column block; row blocks 0 and 2 of a wavefront (lanes 0-15 and
    // 32-47) are the neighbours 2h and 2h + 1, as are row blocks 1 and 3
    const int tx = threadIdx.x & 15, tyl = (threadIdx.x >> 4) & 3, wave = threadIdx.x >> 6;
    const int ty = 2 * (2 * wave + (tyl & 1)) + (tyl >> 1);
    const float s = QUANT ? *scale : 1.0f;

    uint2 rowb[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const size_t idx = static_cast<size_t>(r0 + ty * 8 + i) * C + c0 + tx * 8;
        rowb[i] = load_row8<QUANT>(in, idx, s);
        if constexpr (DUAL) store_stream8(straight + idx, rowb[i]);
    }
    // columns 0..3 come from the .x words, 4..7 from the .y words; rows 0..3 and 4..7 give the two dwords
    const bool odd = tx & 1;
    uint8_t* wr = &tile[(tx * 8) * kPitch + ((((ty >> 1) ^ (tx >> 1)) << 4) | ((ty & 1) << 3))];
    uint32_t lo[4], hi[4];
    transpose4x4(rowb[0].x, rowb[1].x, rowb[2].x, rowb[3].x, lo);
    transpose4x4(rowb[4].x, rowb[5].x, rowb[6].x, rowb[7].x, hi);
#pragma unroll
    for (int j = 0; j < 4; ++j)         // instruction j stores column j ^ odd
        *reinterpret_cast<uint2*>(wr + ((j ^ (odd ? 1 : 0)) * kPitch)) = make_uint2(odd ? lo[j ^ 1] : lo[j], odd ? hi[j ^ 1] : hi[j]);
    transpose4x4(rowb[0].y, rowb[1].y, rowb[2].y, rowb[3].y, lo);
    transpose4x4(rowb[4].y, rowb[5].y, rowb[6].y, rowb[7].y, hi);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uint2*>(wr + ((4 + (j ^ (odd ? 1 : 0))) * kPitch)) = make_uint2(odd ? lo[j ^ 1] : lo[j], odd ? hi[j ^ 1] : hi[j]);
    __syncthreads();

    const int chunk = threadIdx.x & 7, rr = threadIdx.x >> 3;     // 8 lanes cover one 128-byte output row
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int c = p * 32 + rr;
        const uint4 v = *reinterpret_cast<const uint4*>(&tile[c * kPitch + ((chunk ^ (c >> 4)) << 4)]);
        store_stream16(outT + static_cast<size_t>(c0 + c) * R + r0 + chunk * 16, v);
    }
}

// Any shape, any alignment.
template <bool QUANT, bool DUAL>
__global__ __launch_bounds__(kThreads) void k_transpose_generic(const void* __restrict__ in,
                                                                uint8_t* __restrict__ straight,
                                                                uint8_t* __restrict__ outT,
                                                                const float* __restrict__ scale, int R, int C) {
    __shared__ uint8_t tile[64][65];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const float s = QUANT ? *scale : 1.0f;
    for (int i = threadIdx.x; i < 64 * 64; i += kThreads) {
        const int r = r0 + (i >> 6), c = c0 + (i & 63);
        uint8_t b = 0;
        if (r < R && c < C) {
            const size_t idx = static_cast<size_t>(r) * C + c;
            if constexpr (QUANT) b = cvt1_fp8<false>(bf16_to_f32(static_cast<const uint16_t*>(in)[idx]) * s);
            else b = static_cast<const uint8_t*>(in)[idx];
            if constexpr (DUAL) straight[idx] = b;
        }
        tile[i >> 6][i & 63] = b;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += kThreads) {
        const int c = c0 + (i >> 6), r = r0 + (i & 63);
        if (r < R && c < C) outT[static_cast<size_t>(c) * R + r] = tile[i & 63][i >> 6];
    }
}

template <bool QUANT, bool DUAL>
int launch_transpose(const void* in, void* straight, void* outT, const float* scale, int R, int C, cf_stream_t st) {
    if (R < 0 || C < 0) return CF_ERR_INVALID_ARG;
    if (R == 0 || C == 0) return CF_OK;
    if (!in || !outT || (QUANT && !scale) || (DUAL && !straight)) return CF_ERR_INVALID_ARG;
    auto* o = static_cast<uint8_t*>(outT);
    auto* d = static_cast<uint8_t*>(straight);
    const bool fast = R % kTile == 0 && C % kTile == 0 && aligned16(in) && aligned16(outT) &&
                      (!DUAL || aligned16(straight));
    if (fast) {
        dim3 grid(C / kTile, R / kTile);
        k_transpose_tiled<QUANT, DUAL><<<grid, kThreads, 0, as_stream(st)>>>(in, d, o, scale, R, C);
    } else {
        dim3 grid((C + 63) / 64, (R + 63) / 64);
        k_transpose_generic<QUANT, DUAL><<<grid, kThreads, 0, as_stream(st)>>>(in, d, o, scale, R, C);
    }
    return launch_status();
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_fp8_quantize_transpose_e4m3(const uint16_t* d_w, void* d_out, const float* d_scale, int K, int N,
                                   cf_stream_t stream) {
    return launch_transpose<true, false>(d_w, nullptr, d_out, d_scale, K, N, stream);
}

int cf_fp8_quant_and_transpose_e4m3(const uint16_t* d_in, void* d_act8_out, void* d_snap_out,
                                    const float* d_scale, int K, int N, cf_stream_t stream) {
    return launch_transpose<true, true>(d_in, d_act8_out, d_snap_out, d_scale, K, N, stream);
}

int cf_transpose_u8(const void* d_in, void* d_out, int rows, int cols, cf_stream_t stream) {
    return launch_transpose<false, false>(d_in, nullptr, d_out, nullptr, rows, cols, stream);
}

}  // extern "C"
