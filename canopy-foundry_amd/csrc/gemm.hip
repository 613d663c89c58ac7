// Scaled FP8 GEMM for gfx950:  C[M,N] = epilogue( (A[M,K] * sa) . (B[N,K] * sb)^T ).
//
// Kernels in this file, in the order a call tries them:
//   k_gemm_nt_ring        the fast path: persistent, operand tiles copied global -> LDS without staging registers
//                         into a ring of five 32 KiB slots, epilogue through an LDS-staged drain (plain, bias,
//                         SiLU-gate, fp32 / bf16 accumulate; per-tensor or per-row x per-channel scales; dense or
//                         grouped per expert).  Needs K % 128 == 0, K >= 256 and a full-width, aligned C.
//   k_gemm_nt             the same tile with register-staged, double-buffered LDS: any K % 16 == 0, any N.
//   k_gemm_nt_block_ring  1 x 128 / 128 x 128 block scales on the persistent structure (eight wavefronts, partial
//                         products folded into running sums every K-tile); k_gemm_nt_block is its staged fallback.
//   k_gemm_nt_naive       one lane per output element: any shape and alignment, and the on-device cross-check.
//
// Common to the tiled kernels: workgroup tile 256 x 256 x 128 (128 x 256 x 128 with block scales), wavefronts own
// 128 x 128 (64 x 64) sub-tiles of v_mfma_f32_32x32x64_f8f6f4 tiles with fp32 accumulators, one barrier per K-tile.
//
// LDS tile layout: [rows][128 bytes], the eight 16-byte chunks of a row are xor-swizzled with
// f(row) = (row ^ (row >> 3)) & 7 (low five row bits only) so both the 16-byte writes (copies or staging stores)
// and the 16-byte operand reads are spread over all banks.
//
// The weight operand goes to the MFMA "A" side and the activation to the "B" side, so a lane ends up holding four
// consecutive OUTPUT COLUMNS of one output row per accumulator quad: the epilogue scales, applies bias / SiLU-gate
// and rounds to bf16 without a transpose.
//
// Workgroup -> tile mapping is XCD aware: consecutive workgroup ids go round-robin to the 8 XCDs, so each XCD is
// given a contiguous range of tiles, walked in 8 (M) x 4 (N) patches whose operands share its own L2.
#include "common.hpp"
#include "internal.hpp"

#include <mutex>
#include <type_traits>

namespace cf {
namespace {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK;               // 32 KiB per operand tile
constexpr int kStageBytes = 2 * kTileBytes;       // X tile + W tile
constexpr int kLdsBytes = 2 * kStageBytes;        // double buffered: 128 KiB
constexpr int kXcds = 8;

enum { EPI_NONE = 0, EPI_BIAS = 1, EPI_SILU_GATE = 2, EPI_ACCUM_F32 = 3, EPI_ACCUM_BF16 = 4, EPI_STORE_F32 = 5 };
enum { SCALE_TENSOR = 0, SCALE_ROWCOL = 1, SCALE_BLOCK = 2, SCALE_ROW = 3 };   // SCALE_ROW: sa per row, sb one scalar (ring kernel)

struct GemmArgs {
    int M, N, K;                 // N = output columns
    const uint8_t* A; int lda;   // activations [M,K]
    const uint8_t* B; int ldb;   // weights [N,K] (gate weights for EPI_SILU_GATE)
    const uint8_t* B2;           // up weights [N,K] for EPI_SILU_GATE
    const float* sa;             // descale of A: [1] or [M]
    const float* sb;             // descale of B: [1] or [N]
    const float* sb2;            // descale of B2
    const uint16_t* bias;        // bf16 [N] for EPI_BIAS
    uint16_t* C; int ldc;        // bf16 [M,N]
    float* Cf;                   // fp32 [M,N] for EPI_ACCUM_F32 (C += product)
    int tiles_m, tiles_n;
    int force_staged;            // take the register-staged kernel even when the ring kernel applies
    int duo;                     // 1: the two-workgroups-per-CU kernel where it applies, 2: the same without the stagger
    int mfma32;                  // keep k_gemm_nt_ring (the 32 x 32 x 64 MFMA shape) where k_gemm_nt_ring16 would apply
    // grouped (per-expert) form, ring kernel only; all null / 0 for a dense GEMM
    const int* tile_map;         // [0] = number of row tiles, then (expert, first row, end row) per row tile
    const int* a_row_index;      // compact row r reads A row (and its descale) a_row_index[r]; null = r
    int a_rows;                  // rows of the A buffer (= M without a row index)
    long long b_expert_stride;   // bytes between the weight matrices of consecutive experts
    int sb_expert_stride;        // elements between the channel descales of consecutive experts
    // term-split form (ring kernel, MX instantiation only): A's K axis is `K / b_k_period` terms laid side by side,
    // term t = the residual of the terms before it scaled by 16^t; every term multiplies the same b_k_period
    // columns of B, and the matrix cores scale its products by 2^(-4 t)
    int b_k_period;
};

// where a workgroup's tile lives: rows [m0, m_end) of the output, columns from n0, weights of `expert`
struct TilePos { int m0, m_end, n0, expert; };

__device__ __forceinline__ int swz(int row) { return (row ^ ((row >> 3) & 3)) & 7; }

// Tile t of the walk order -> (tile_m, tile_n): patches of 8 (M) x tiles_n, row tiles varying fastest, so that
// 32 consecutive tiles form an 8 x 4 patch whose operands an XCD's L2 can hold.
__device__ __forceinline__ void tile_coords(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
    constexpr int GM = 8;
    const int group = t / (GM * tiles_n);
    const int first_m = group * GM;
    const int gm = min(GM, tiles_m - first_m);
    const int in_group = t - group * GM * tiles_n;
    tm = first_m + in_group % gm;
    tn = in_group / gm;
}
// Workgroups are handed to the 8 XCDs round-robin, so launch positions with the same pos % 8 share an XCD
// (and its L2).  One tile per workgroup: position pos works on tile (pos % 8) * (total / 8) + pos / 8 of the walk
// order, so each XCD is given a contiguous range of tiles (ragged counts keep the plain order).
__device__ __forceinline__ int xcd_chunked(int pos, int total) {
    return total % kXcds == 0 ? (pos % kXcds) * (total / kXcds) + pos / kXcds : pos;
}

// ---- epilogue shared by the tiled kernels ----------------------------------------
// acc[a][b][r]: output row m = m0 + wm*128 + b*32 + (lane & 31); weight row within the
// wave's 128 = a*32 + 8*(r/4) + 4*(lane>>5) + r%4, i.e. four consecutive output columns per quad.
// Column scales are fetched once per quad as a float4 and reused for the four row tiles.

// SiLU gate for the fused epilogue: x * 1/(1 + 2^(-x*log2 e)) on the hardware exp2 and reciprocal
// (1 ulp each).  The stand-alone swiglu kernel keeps the correctly-rounded divide and the
// reproducible expf; the two differ by at most one bf16 ulp of the product.
__device__ __forceinline__ float fast_silu(float x) {
    const float e = __builtin_amdgcn_exp2f(-1.44269504f * x);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float4 load_scale4(const float* s, int n, int N, bool fast) {
    if (fast) return *reinterpret_cast<const float4*>(s + n);
    return make_float4(s[min(n, N - 1)], s[min(n + 1, N - 1)], s[min(n + 2, N - 1)], s[min(n + 3, N - 1)]);
}

template <int EPI, int SCALE>
__device__ __forceinline__ void epilogue(v16f (&acc)[4][4], const GemmArgs& p, int m0, int n0, int wm, int wn,
                                         int lane) {
    const int khalf = lane >> 5;
    constexpr bool GATE = EPI == EPI_SILU_GATE;
    constexpr int NT = GATE ? 2 : 4;                       // 32-wide output column tiles per wave
    const int nbase = n0 + wn * (NT * 32) + khalf * 4;     // + t*32 + g*8
    const bool vec_ok = EPI == EPI_ACCUM_F32 ? (p.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.Cf) & 15u) == 0)
                                             : (p.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 7u) == 0);
    const bool full_n = n0 + (GATE ? BN / 2 : BN) <= p.N;

    float s1 = 0.0f, s2 = 0.0f;
    if constexpr (SCALE == SCALE_TENSOR) {
        s1 = p.sa[0] * p.sb[0];
        if constexpr (GATE) s2 = p.sa[0] * p.sb2[0];
    }
    const bool fast = SCALE != SCALE_TENSOR && full_n && ((reinterpret_cast<uintptr_t>(p.sb) & 15u) == 0) &&
                      (!GATE || (reinterpret_cast<uintptr_t>(p.sb2) & 15u) == 0);
    // row factors and row validity of this lane's four output rows
    float sa[4];
    int mrow[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        mrow[b] = m0 + wm * 128 + b * 32 + (lane & 31);
        if constexpr (SCALE == SCALE_TENSOR) {
            sa[b] = 1.0f;
        } else {
            const int r = min(mrow[b], p.M - 1);
            sa[b] = p.sa[p.a_row_index ? p.a_row_index[r] : r];
        }
    }

#pragma unroll
    for (int t = 0; t < NT; ++t) {
        // per-quad column factors of this 32-column tile: [g] -> 4 columns
        float4 cs[4], cs2[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if constexpr (SCALE == SCALE_TENSOR) {
                cs[g] = make_float4(s1, s1, s1, s1);
                cs2[g] = make_float4(s2, s2, s2, s2);
            } else {
                cs[g] = load_scale4(p.sb, nbase + t * 32 + g * 8, p.N, fast);
                if constexpr (GATE) cs2[g] = load_scale4(p.sb2, nbase + t * 32 + g * 8, p.N, fast);
            }
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int m = mrow[b];
            if (m >= p.M) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = nbase + t * 32 + g * 8;
                const float c4[4] = {cs[g].x, cs[g].y, cs[g].z, cs[g].w};
                if constexpr (EPI == EPI_ACCUM_F32) {
                    // beta = 1: the product is added to what the caller's fp32 buffer holds
                    float* frow = p.Cf + static_cast<size_t>(m) * p.ldc + n;
                    if (vec_ok && n + 3 < p.N) {
                        float4 v = *reinterpret_cast<const float4*>(frow);
                        v.x += acc[t][b][g * 4 + 0] * c4[0];
                        v.y += acc[t][b][g * 4 + 1] * c4[1];
                        v.z += acc[t][b][g * 4 + 2] * c4[2];
                        v.w += acc[t][b][g * 4 + 3] * c4[3];
                        *reinterpret_cast<float4*>(frow) = v;
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; ++q) if (n + q < p.N) frow[q] += acc[t][b][g * 4 + q] * c4[q];
                    }
                } else {
                    uint16_t* crow = p.C + static_cast<size_t>(m) * p.ldc + n;
                    float v[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if constexpr (GATE) {
                            const float u4[4] = {cs2[g].x, cs2[g].y, cs2[g].z, cs2[g].w};
                            // the reference rounds gate and up to bf16 before the SiLU product
                            const float gate = round_bf16_hw(acc[2 * t][b][g * 4 + q] * (sa[b] * c4[q]));
                            const float up = round_bf16_hw(acc[2 * t + 1][b][g * 4 + q] * (sa[b] * u4[q]));
                            v[q] = fast_silu(gate) * up;
                        } else {
                            v[q] = acc[t][b][g * 4 + q] * (sa[b] * c4[q]);
                            if constexpr (EPI == EPI_ACCUM_BF16) {
                                if (n + q < p.N) v[q] += bf16_to_f32(crow[q]);
                            }
                            if constexpr (EPI == EPI_BIAS)   // bias is added to the bf16 result, as the separate kernel does
                                v[q] = round_bf16_hw(v[q]) + bf16_to_f32(p.bias[min(n + q, p.N - 1)]);
                        }
                    }
                    const uint32_t o01 = pack_bf16x2_hw(v[0], v[1]), o23 = pack_bf16x2_hw(v[2], v[3]);
                    if (vec_ok && n + 3 < p.N) {
                        *reinterpret_cast<uint2*>(crow) = make_uint2(o01, o23);
                    } else {
                        const uint16_t o[4] = {(uint16_t)(o01 & 0xffffu), (uint16_t)(o01 >> 16), (uint16_t)(o23 & 0xffffu), (uint16_t)(o23 >> 16)};
#pragma unroll
                        for (int q = 0; q < 4; ++q) if (n + q < p.N) crow[q] = o[q];
                    }
                }
            }
            // keep the scheduler from pulling every accumulator into VGPRs at once: in the persistent
            // kernel the next tile's operands are live across the epilogue
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// FMT bit 0: A (activation side) is E5M2; bit 1: B (weight side) is E5M2
template <int FMT, int EPI, int SCALE>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void k_gemm_nt(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    int tile_m, tile_n;
    tile_coords(xcd_chunked(blockIdx.x, p.tiles_m * p.tiles_n), p.tiles_m, p.tiles_n, tile_m, tile_n);
    constexpr int OUT_BN = EPI == EPI_SILU_GATE ? BN / 2 : BN;     // output columns per workgroup
    const int m0 = tile_m * BM, n0 = tile_n * OUT_BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> register staging: thread owns chunk c of rows r0 + 32 i ----
    const int r0 = tid >> 3, c = tid & 7;
    const int lds_w = r0 * BK + ((c ^ swz(r0)) << 4);
    const uint8_t* xsrc[8];
    const uint8_t* wsrc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = r0 + 32 * i;
        xsrc[i] = p.A + static_cast<size_t>(min(m0 + row, p.M - 1)) * p.lda + c * 16;
        if constexpr (EPI == EPI_SILU_GATE) {
            // LDS weight rows of a wave: [gate 32 | up 32 | gate 32 | up 32] over the same 64 output columns
            const int t = (row >> 5) & 3, w = row >> 7;
            const int n = n0 + w * 64 + (t >> 1) * 32 + (row & 31);
            wsrc[i] = ((t & 1) ? p.B2 : p.B) + static_cast<size_t>(min(n, p.N - 1)) * p.ldb + c * 16;
        } else {
            wsrc[i] = p.B + static_cast<size_t>(min(n0 + row, p.N - 1)) * p.ldb + c * 16;
        }
    }
    const bool kfull = (p.K % BK) == 0;
    uint4 xr[8], wr[8];
    auto fetch = [&](int k0) {
        const bool live = kfull || (k0 + c * 16 < p.K);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            xr[i] = live ? *reinterpret_cast<const uint4*>(xsrc[i] + k0) : make_uint4(0, 0, 0, 0);
            wr[i] = live ? *reinterpret_cast<const uint4*>(wsrc[i] + k0) : make_uint4(0, 0, 0, 0);
        }
    };
    auto stash = [&](int stage) {
        uint8_t* xs = smem + stage * kStageBytes + lds_w;
        uint8_t* ws = xs + kTileBytes;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            *reinterpret_cast<uint4*>(xs + i * 32 * BK) = xr[i];
            *reinterpret_cast<uint4*>(ws + i * 32 * BK) = wr[i];
        }
    };

    // ---- LDS -> MFMA operand addressing ----
    const int frow = lane & 31, khalf = lane >> 5, fs = swz(frow);
    int rd[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int j = 0; j < 2; ++j) rd[s][j] = frow * BK + (((s * 4 + khalf * 2 + j) ^ fs) << 4);
    const int x_base = wm * 128 * BK, w_base = kTileBytes + wn * 128 * BK;

    v16f acc[4][4];   // [weight tile][activation tile]
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    const int ktiles = (p.K + BK - 1) / BK;
    fetch(0);
    stash(0);
    __syncthreads();

    for (int kt = 0; kt < ktiles; ++kt) {
        const int stage = kt & 1;
        const bool more = kt + 1 < ktiles;
        if (more) fetch((kt + 1) * BK);
        const uint8_t* st = smem + stage * kStageBytes;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            v8i wf[4], xf[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint4 w0 = *reinterpret_cast<const uint4*>(st + w_base + t * 32 * BK + rd[s][0]);
                const uint4 w1 = *reinterpret_cast<const uint4*>(st + w_base + t * 32 * BK + rd[s][1]);
                wf[t] = v8i{(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
                const uint4 x0 = *reinterpret_cast<const uint4*>(st + x_base + t * 32 * BK + rd[s][0]);
                const uint4 x1 = *reinterpret_cast<const uint4*>(st + x_base + t * 32 * BK + rd[s][1]);
                xf[t] = v8i{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
            }
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                        wf[a], xf[b], acc[a][b], (FMT >> 1) & 1 /* weight side */, FMT & 1 /* activation side */, 0, 0, 0, 0);
        }
        if (more) stash(stage ^ 1);
        __syncthreads();
    }

    epilogue<EPI, SCALE>(acc, p, m0, n0, wm, wn, lane);
}


// ---- block-scaled kernel: activation scales per 1 x 128 K-group, weight scales per 128 x 128 block ----
// Workgroup tile 128 x 256 x 128, four wavefronts 2 x 2, each 64 x 128 = 4 x 2 MFMA tiles.  One K-tile
// is exactly one scale group, so each K-tile is multiplied into a zeroed set of partial accumulators
// (128 registers) and then promoted into the running sum with the group's factor
// sa[m, kt] * sb[n / 128, kt] on the vector ALU (another 128 registers).  Register-staged loads,
// double-buffered LDS, one barrier per K-tile; K is zero-padded up to a multiple of 128.
constexpr int BSM = 128;                                   // rows per workgroup
constexpr int kBlkX = BSM * BK, kBlkW = BN * BK;           // 16 KiB + 32 KiB per stage
constexpr int kBlkStage = kBlkX + kBlkW;
constexpr int kBlkLds = 2 * kBlkStage;                     // 96 KiB

__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void k_gemm_nt_block(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // plain order with 8-row groups: the block-scaled shapes are modest and L2 resident
    const int tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
    const int m0 = tile_m * BSM, n0 = tile_n * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kb = (p.K + BK - 1) / BK;                    // scale groups along K

    const int r0 = tid >> 3, c = tid & 7;
    const int lds_w = r0 * BK + ((c ^ swz(r0)) << 4);
    const uint8_t* xsrc[4];
    const uint8_t* wsrc[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) xsrc[i] = p.A + static_cast<size_t>(min(m0 + r0 + 32 * i, p.M - 1)) * p.lda + c * 16;
#pragma unroll
    for (int i = 0; i < 8; ++i) wsrc[i] = p.B + static_cast<size_t>(min(n0 + r0 + 32 * i, p.N - 1)) * p.ldb + c * 16;
    uint4 xr[4], wr[8];
    auto fetch = [&](int k0) {
        const bool live = k0 + c * 16 < p.K;
#pragma unroll
        for (int i = 0; i < 4; ++i) xr[i] = live ? *reinterpret_cast<const uint4*>(xsrc[i] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 8; ++i) wr[i] = live ? *reinterpret_cast<const uint4*>(wsrc[i] + k0) : make_uint4(0, 0, 0, 0);
    };
    auto stash = [&](int stage) {
        uint8_t* xs = smem + stage * kBlkStage + lds_w;
        uint8_t* ws = xs + kBlkX;
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(xs + i * 32 * BK) = xr[i];
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(ws + i * 32 * BK) = wr[i];
    };

    const int frow = lane & 31, khalf = lane >> 5, fs = swz(frow);
    int rd[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int j = 0; j < 2; ++j) rd[s][j] = frow * BK + (((s * 4 + khalf * 2 + j) ^ fs) << 4);
    const int x_base = wm * 64 * BK, w_base = kBlkX + wn * 128 * BK;

    v16f sum[4][2];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) sum[a][b][r] = 0.0f;

    // this lane's two output rows and this wave's weight block row
    int mrow[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) mrow[b] = min(m0 + wm * 64 + b * 32 + (lane & 31), p.M - 1);
    const int nblk = min(n0 + wn * 128, p.N - 1) / 128;

    fetch(0);
    stash(0);
    __syncthreads();
    for (int kt = 0; kt < kb; ++kt) {
        const int stage = kt & 1;
        const bool more = kt + 1 < kb;
        if (more) fetch((kt + 1) * BK);
        // the group's factors: issued before the MFMAs so they have landed when the promotion needs them
        const float sbv = p.sb[static_cast<size_t>(nblk) * kb + kt];
        float f[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) f[b] = p.sa[static_cast<size_t>(mrow[b]) * kb + kt] * sbv;
        const uint8_t* st = smem + stage * kBlkStage;
        v16f part[4][2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            v8i wf[4], xf[2];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint4 w0 = *reinterpret_cast<const uint4*>(st + w_base + t * 32 * BK + rd[s][0]);
                const uint4 w1 = *reinterpret_cast<const uint4*>(st + w_base + t * 32 * BK + rd[s][1]);
                wf[t] = v8i{(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint4 x0 = *reinterpret_cast<const uint4*>(st + x_base + t * 32 * BK + rd[s][0]);
                const uint4 x1 = *reinterpret_cast<const uint4*>(st + x_base + t * 32 * BK + rd[s][1]);
                xf[t] = v8i{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
            }
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    v16f cin;
                    if (s == 0) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) cin[r] = 0.0f;
                    } else {
                        cin = part[a][b];
                    }
                    part[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[a], xf[b], cin, 0, 0, 0, 0, 0, 0);
                }
        }
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum[a][b][r] = __builtin_fmaf(part[a][b][r], f[b], sum[a][b][r]);
        if (more) stash(stage ^ 1);
        __syncthreads();
    }

    // epilogue: the sums are already scaled; lane holds four consecutive columns per quad
    const bool vec_ok = (p.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 7u) == 0);
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int m = m0 + wm * 64 + b * 32 + (lane & 31);
        if (m >= p.M) continue;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * 128 + a * 32 + g * 8 + khalf * 4;
                uint16_t* crow = p.C + static_cast<size_t>(m) * p.ldc + n;
                const uint32_t o01 = pack_bf16x2_hw(sum[a][b][g * 4 + 0], sum[a][b][g * 4 + 1]);
                const uint32_t o23 = pack_bf16x2_hw(sum[a][b][g * 4 + 2], sum[a][b][g * 4 + 3]);
                if (vec_ok && n + 3 < p.N) {
                    *reinterpret_cast<uint2*>(crow) = make_uint2(o01, o23);
                } else {
                    const uint16_t o[4] = {(uint16_t)(o01 & 0xffffu), (uint16_t)(o01 >> 16), (uint16_t)(o23 & 0xffffu), (uint16_t)(o23 >> 16)};
#pragma unroll
                    for (int q = 0; q < 4; ++q) if (n + q < p.N) crow[q] = o[q];
                }
            }
    }
}

// ---- ring kernel: direct-to-LDS copies into five 32 KiB slots --------------------------------
// Needs K % 128 == 0, K >= 256 and operands smaller than 4 GiB.  global_load_lds_dwordx4 copies
// 16 bytes per lane from global memory straight into LDS (lane l lands at base + 16*l): no staging
// registers, and eight lanes fetch one full 128-byte line of a row (half-line requests reach only
// ~60% of the L2 rate).  The copies take a uniform 64-bit base (operand + K offset, scalar registers)
// plus a 32-bit per-lane byte offset, so advancing along K costs two scalar adds per K-tile.
// A slot holds one operand tile [256 rows][128 bytes], chunks xor-swizzled as in the staged kernel.
// Operand tile i (X of K-tile i/2 for even i, W for odd i) lives in slot i % 5, so while K-tile kt is
// being multiplied, K-tile kt+1 is resident or landing and the X half of kt+2 is already on its way.
// The five slot offsets are carried as a rotating set of scalars (no division in the loop).
//
// A K-tile is two MFMA steps (k-halves of 64).  Step (kt,0): 16 MFMAs, the operand reads of (kt,1),
// the 8 copies of X(kt+2).  Step (kt,1): 2 MFMAs, wait for K-tile kt+1, barrier, 14 MFMAs woven
// with the operand reads of (kt+1,0) and the 8 copies of W(kt+2).  One barrier per 2048 MFMA cycles;
// a copy has two to three steps (2000-3000 cycles) to land.  With one wavefront per SIMD an
// instruction issues every four cycles at best, so everything between two MFMAs (64 cycles) is kept
// to a handful of instructions.
constexpr int kSlotBytes = BM * BK;               // 32 KiB
constexpr int kSlots = 5;
constexpr int kRingLds = kSlots * kSlotBytes;     // 160 KiB: all of a CU's LDS

// s_waitcnt immediates: vmcnt in bits [3:0] and [15:14], expcnt [6:4] and lgkmcnt [11:8] left at no-wait
constexpr int kWaitVm0 = 0x0f70, kWaitVm8 = 0x0f78, kWaitVm16 = 0x4f70;

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Tile `lin` of a workgroup's walk order -> where it lives.  Dense: the patch order of tile_coords.  Grouped:
// the table holds, per row tile, its expert's number, row range, first row tile and row-tile count, experts back
// to back; an expert's tiles are walked in groups of 4 column tiles with its row tiles varying fastest, so that
// 32 consecutive tiles are (up to) 8 row tiles x 4 column tiles of one expert.
constexpr int kMapWords = 5;
template <int OUT_BN>
__device__ __forceinline__ TilePos locate_tile(const GemmArgs& p, int lin) {
    TilePos t;
    if (p.tile_map) {
        const int* e = p.tile_map + 1 + kMapWords * (lin / p.tiles_n);
        const int expert = e[0], row_base = e[1], row_end = e[2], first_rt = e[3], n_rt = e[4];
        constexpr int GN = 4;
        const int local = lin - first_rt * p.tiles_n;
        const int g = local / (n_rt * GN);
        const int within = local - g * n_rt * GN;
        const int rt = within % n_rt;
        t.expert = expert;
        t.m0 = row_base + rt * BM;
        t.m_end = min(t.m0 + BM, row_end);
        t.n0 = (g * GN + within / n_rt) * OUT_BN;
    } else {
        int tile_m, tile_n;
        tile_coords(lin, p.tiles_m, p.tiles_n, tile_m, tile_n);
        t.expert = 0;
        t.m0 = tile_m * BM;
        t.m_end = p.M;
        t.n0 = tile_n * OUT_BN;
    }
    return t;
}

// Drain of a tile.  A unit is 32 output columns: one accumulator column of the wavefront (gate and up
// accumulators of the same columns for the SiLU-gate epilogue); units are drained in pairs (64 columns =
// one 128-byte line of bf16 per row).  TileScales holds what the drain needs in registers: the descales
// of this lane's four output rows, and the channel descales of the pair being drained (cs[u][g] = the
// four consecutive columns of accumulator quad g of unit u); the next pair's are fetched while the
// current one is drained, the first pair's while the tile's last MFMAs run.
template <int EPI>
struct TileScales {
    float sa[4];
    float4 cs[2][4];
    float4 cs2[2][4];      // up-projection descales (SiLU-gate)
};

template <int EPI, int SCALE>
__device__ __forceinline__ void load_row_scales(TileScales<EPI>& s, const GemmArgs& p, const TilePos& t, int wm, int lane) {
    if constexpr (SCALE == SCALE_ROWCOL || SCALE == SCALE_ROW) {
        // Two complete paths: these loads are issued among the copies of the tile's last K-tile, and a wait between
        // a row-index load and the scale load that depends on it also waits for every copy in flight.  Without a
        // row index nothing waits; with one, the four index loads share a single wait.
        int r[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) r[b] = min(t.m0 + wm * 128 + b * 32 + (lane & 31), t.m_end - 1);
        if (p.a_row_index) {
#pragma unroll
            for (int b = 0; b < 4; ++b) r[b] = p.a_row_index[r[b]];
#pragma unroll
            for (int b = 0; b < 4; ++b) s.sa[b] = p.sa[r[b]];
            asm volatile("; row scales through the row index" ::: "memory");      // keeps the two paths from being merged again
        } else {
#pragma unroll
            for (int b = 0; b < 4; ++b) s.sa[b] = p.sa[r[b]];
        }
    }
}
template <int EPI, int SCALE>
__device__ __forceinline__ void load_pair_scales(float4 (&cs)[2][4], float4 (&cs2)[2][4], const GemmArgs& p,
                                                 const TilePos& t, int wn, int lane, int pair) {
    constexpr int NU = EPI == EPI_SILU_GATE ? 2 : 4;
    // uniform bases (scalar registers) + a small per-lane byte offset: no 64-bit per-lane addresses to keep alive
    const size_t col0 = t.n0 + wn * (NU * 32) + pair * 64;
    if constexpr (SCALE == SCALE_ROWCOL) {
        const size_t ucol = static_cast<size_t>(t.expert) * p.sb_expert_stride + col0;
        const uint8_t* b1 = reinterpret_cast<const uint8_t*>(p.sb + ucol);
        const uint8_t* b2 = reinterpret_cast<const uint8_t*>(EPI == EPI_SILU_GATE ? p.sb2 + ucol : p.sb);
        const uint32_t loff = static_cast<uint32_t>(lane >> 5) * 16u;
        if constexpr (EPI != EPI_SILU_GATE) {
            // a last column tile that N cuts short (N % 4 == 0): factors of columns at or beyond N are not used,
            // their loads are moved onto the last four columns
            if (t.n0 + BN > p.N) {
                const int lim = (p.N - 4 - static_cast<int>(t.n0 + wn * (NU * 32) + pair * 64)) * 4;
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        cs[u][g] = *reinterpret_cast<const float4*>(b1 + min(static_cast<int>(loff + u * 128u + g * 32u), lim));
                return;
            }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                cs[u][g] = *reinterpret_cast<const float4*>(b1 + (loff + u * 128u + g * 32u));
                if constexpr (EPI == EPI_SILU_GATE) cs2[u][g] = *reinterpret_cast<const float4*>(b2 + (loff + u * 128u + g * 32u));
            }
    }
}

// An accumulator element as a VALU operand.  The explicit AGPR read keeps the register allocator from
// moving whole accumulator tiles into VGPRs (and from there to scratch) around the drain.
__device__ __forceinline__ float acc_read(float a) {
    float v;
    asm("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}

// Per pair of units and per 64 output rows the wavefront scales its accumulators, applies the epilogue,
// rounds to bf16 and parks the 64 rows x 128 bytes in its own 8 KiB of a free ring slot (16-byte chunks
// xor-swizzled by row: two-pass ds_write_b64, conflict-free ds_read_b128), then streams them out 16 bytes
// per lane, eight lanes per row, so that every store instruction writes whole 128-byte lines.  The stores
// are non-temporal: the output is not read again here and should not displace operand tiles from L2.
// RAGGED: the tile may end before its 256th row; rows at or beyond t.m_end are then not stored.
template <int EPI, int SCALE, bool RAGGED, class Landed>
__device__ __forceinline__ void drain_tile(v16f (&acc)[4][4], TileScales<EPI>& s, float s1, float s2, const GemmArgs& p,
                                           const TilePos& t, int wm, int wn, int lane, uint8_t* stage, Landed&& landed) {
    constexpr bool GATE = EPI == EPI_SILU_GATE;
    constexpr int NU = GATE ? 2 : 4;
    const int row = lane & 31, khalf = lane >> 5;
    uint8_t* wr = stage + row * 128 + khalf * 8;
    const int wswz = (row >> 1) & 7;
    const int rr = lane >> 3, rc = lane & 7;
    // row rr + 8 i sits at swizzle (rr >> 1) ^ 4 (i & 1): two read bases, even and odd i
    const uint8_t* rdp0 = stage + rr * 128 + ((rc ^ (rr >> 1)) << 4);
    const uint8_t* rdp1 = stage + rr * 128 + ((rc ^ (rr >> 1) ^ 4) << 4);
    const int mrow0 = t.m0 + wm * 128 + rr;
    // stores: uniform base per pair and 8-row group (scalar registers) + this lane's byte offset
    uint8_t* cu = reinterpret_cast<uint8_t*>(p.C + static_cast<size_t>(t.m0 + wm * 128) * p.ldc + t.n0 + wn * (NU * 32));
    const uint32_t coff = (static_cast<uint32_t>(rr) * static_cast<uint32_t>(p.ldc) + rc * 8u) * 2u;
    const size_t cstep = static_cast<size_t>(p.ldc) * 16;      // bytes between 8-row groups
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    // Bias is added to the bf16 result, as the separate kernel does: on the way out, where a lane holds eight
    // consecutive columns of a row, the same eight for every row it stores.  Both pairs' bias chunks are
    // fetched before the first store, so no wait on them has to sit out a store burst.
    uint4 bias8[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
    if constexpr (EPI == EPI_BIAS) {
        const int bcol = t.n0 + wn * (NU * 32) + rc * 8;
#pragma unroll
        for (int pair = 0; pair < NU / 2; ++pair)
            bias8[pair] = *reinterpret_cast<const uint4*>(p.bias + (RAGGED ? min(bcol + pair * 64, p.N - 8) : bcol + pair * 64));
    }
    // RAGGED also covers a last column tile that N cuts short (N % 8 == 0): this lane's eight columns of a pair
    // are stored or not as a whole
    const int ncol0 = t.n0 + wn * (NU * 32) + rc * 8;

#pragma unroll
    for (int pair = 0; pair < NU / 2; ++pair) {
        const uint4 bv = bias8[pair];
        const float bf[8] = {bf16_lo(bv.x), bf16_hi(bv.x), bf16_lo(bv.y), bf16_hi(bv.y),
                             bf16_lo(bv.z), bf16_hi(bv.z), bf16_lo(bv.w), bf16_hi(bv.w)};
        // the next pair's factors are fetched while this pair is drained
        float4 ncs[2][4], ncs2[2][4];
        if (pair + 1 < NU / 2) load_pair_scales<EPI, SCALE>(ncs, ncs2, p, t, wn, lane, pair + 1);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int bb = 0; bb < 2; ++bb) {
                const int b = half * 2 + bb;
                const float sa = (SCALE == SCALE_ROWCOL || SCALE == SCALE_ROW) ? s.sa[b] : 1.0f;
#pragma unroll
                for (int uu = 0; uu < 2; ++uu) {
                    const int unit = pair * 2 + uu;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        float4 c = make_float4(s1, s1, s1, s1), u = make_float4(s2, s2, s2, s2);
                        if constexpr (SCALE == SCALE_ROWCOL) {
                            c = s.cs[uu][g];
                            if constexpr (GATE) u = s.cs2[uu][g];
                        }
                        const float c4[4] = {c.x, c.y, c.z, c.w}, u4[4] = {u.x, u.y, u.z, u.w};
                        float v[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            if constexpr (GATE) {
                                // the reference rounds gate and up to bf16 before the SiLU product: one conversion
                                // instruction rounds both
                                const uint32_t gu = pack_bf16x2_hw(acc_read(acc[2 * unit][b][g * 4 + q]) * (sa * c4[q]),
                                                                   acc_read(acc[2 * unit + 1][b][g * 4 + q]) * (sa * u4[q]));
                                v[q] = fast_silu(bf16_lo(gu)) * bf16_hi(gu);
                            } else {
                                v[q] = acc_read(acc[unit][b][g * 4 + q]) * (sa * c4[q]);
                            }
                        }
                        *reinterpret_cast<uint2*>(wr + bb * 32 * 128 + (((uu * 4 + g) ^ wswz) << 4)) =
                            make_uint2(pack_bf16x2_hw(v[0], v[1]), pack_bf16x2_hw(v[2], v[3]));
                    }
                    __builtin_amdgcn_sched_barrier(0);     // one accumulator (pair) in flight at a time: keeps the drain in few registers
                }
            }
            // Stores and copies share one completion counter, and a wait on copies issued after these stores
            // would have to sit out the whole burst.  So the K-tile still landing is waited for here, where it
            // costs next to nothing (its copies are older than a quarter of the drain's work), and the tile
            // that follows skips the wait of its first K-tile: the stores then have two K-tiles to complete.
            if (pair == 0 && half == 0) {
                __builtin_amdgcn_s_waitcnt(kWaitVm0);
                landed();                      // the caller's loads that must not meet copies in flight
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint4 v = *reinterpret_cast<const uint4*>(((i & 1) ? rdp1 : rdp0) + i * 8 * 128);
                if constexpr (EPI == EPI_BIAS) {
                    v.x = pack_bf16x2_hw(bf16_lo(v.x) + bf[0], bf16_hi(v.x) + bf[1]);
                    v.y = pack_bf16x2_hw(bf16_lo(v.y) + bf[2], bf16_hi(v.y) + bf[3]);
                    v.z = pack_bf16x2_hw(bf16_lo(v.z) + bf[4], bf16_hi(v.z) + bf[5]);
                    v.w = pack_bf16x2_hw(bf16_lo(v.w) + bf[6], bf16_hi(v.w) + bf[7]);
                }
                if (!RAGGED || (mrow0 + half * 64 + i * 8 < t.m_end && ncol0 + pair * 64 < p.N)) {
                    const u32x4 vv = {v.x, v.y, v.z, v.w};
                    __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>(cu + ((half * 8 + i) * cstep + pair * 128) + coff));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (pair + 1 < NU / 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int g = 0; g < 4; ++g) { s.cs[u][g] = ncs[u][g]; s.cs2[u][g] = ncs2[u][g]; }
        }
    }
}

// The accumulate forms (C += product, per-tensor scale s1; C fp32, or bf16 with one rounding of the sum): per pair
// of units and per 32 output rows the scaled accumulators are parked as 32 rows x 256 bytes of fp32 (chunks
// xor-swizzled by row), read back 16 bytes per lane, sixteen lanes per row, added to what C holds (fetched while
// the block is being scaled) and stored: whole lines in both directions (128 bytes of fp32, 64 of bf16 per
// sixteen lanes), non-temporal both ways.
// STORE: C = product (nothing is fetched).  RAGGED also covers a last column tile that N cuts short (N % 4 == 0: a
// lane's four columns are in or out as a whole).
// sa: the descales of this lane's four output rows (1 for the per-tensor forms), s1 the scalar factor.
template <bool RAGGED, bool OUT_BF16, bool STORE, class Landed>
__device__ __forceinline__ void drain_tile_accum(v16f (&acc)[4][4], const float (&sa)[4], float s1, const GemmArgs& p, const TilePos& t,
                                                 int wm, int wn, int lane, uint8_t* stage, Landed&& landed) {
    const int row = lane & 31, khalf = lane >> 5;
    uint8_t* wr = stage + row * 256;
    const int wswz = row & 15;
    const int rr = lane >> 4, rc = lane & 15;
    const int mrow0 = t.m0 + wm * 128 + rr;
    const int ncol0 = t.n0 + wn * 128 + rc * 4;                 // + 64 per pair
    constexpr uint32_t ES = OUT_BF16 ? 2u : 4u;                 // bytes per element of C
    const size_t c_first = static_cast<size_t>(t.m0 + wm * 128) * p.ldc + t.n0 + wn * 128;
    uint8_t* cu = OUT_BF16 ? reinterpret_cast<uint8_t*>(p.C + c_first) : reinterpret_cast<uint8_t*>(p.Cf + c_first);
    const uint32_t coff = (static_cast<uint32_t>(rr) * static_cast<uint32_t>(p.ldc) + rc * 4u) * ES;
    const size_t cstep = static_cast<size_t>(p.ldc) * 4 * ES;   // bytes between 4-row groups
    constexpr uint32_t pair_bytes = 64 * ES;                    // a pair of units is 64 columns
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

    // What C holds is fetched DEPTH blocks (of 32 rows x 64 columns) ahead of its use: every fetch pays the full
    // memory latency (all workgroups drain at the same moment), so the first blocks are requested before anything
    // else and the later ones as the registers of the earlier ones come free.
    using Raw = std::conditional_t<OUT_BF16, u32x2, f32x4>;
    constexpr int DEPTH = OUT_BF16 ? 4 : 2;      // what the register budget allows beside the copy offsets
    Raw old[DEPTH][8];
    auto fetch_old = [&](auto kc) {
        constexpr int k = decltype(kc)::value, pair = k >> 2, b = k & 3;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            old[k % DEPTH][i] = Raw{};
            if (!STORE && (!RAGGED || (mrow0 + b * 32 + i * 4 < t.m_end && ncol0 + pair * 64 < p.N)))
                old[k % DEPTH][i] = __builtin_nontemporal_load(reinterpret_cast<const Raw*>(cu + ((b * 8 + i) * cstep + pair * pair_bytes) + coff));
        }
    };
    if constexpr (!STORE) static_for<0, DEPTH>([&](auto kc) { fetch_old(kc); });

    static_for<0, 8>([&](auto kc) {
        constexpr int k = decltype(kc)::value, pair = k >> 2, b = k & 3;
#pragma unroll
        for (int uu = 0; uu < 2; ++uu) {
            const int unit = pair * 2 + uu;
            const float sr = sa[b] * s1;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float4 v;
                v.x = acc_read(acc[unit][b][g * 4 + 0]) * sr;
                v.y = acc_read(acc[unit][b][g * 4 + 1]) * sr;
                v.z = acc_read(acc[unit][b][g * 4 + 2]) * sr;
                v.w = acc_read(acc[unit][b][g * 4 + 3]) * sr;
                *reinterpret_cast<float4*>(wr + (((uu * 8 + g * 2 + khalf) ^ wswz) << 4)) = v;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // as in drain_tile: every copy in flight is waited for before the first store, and the tile that
        // follows skips the wait of its first K-tile
        if constexpr (k == 0) {
            __builtin_amdgcn_s_waitcnt(kWaitVm0);
            landed();
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = i * 4 + rr;
            const float4 v = *reinterpret_cast<const float4*>(stage + r * 256 + ((rc ^ (r & 15)) << 4));
            if (!RAGGED || (mrow0 + b * 32 + i * 4 < t.m_end && ncol0 + pair * 64 < p.N)) {
                uint8_t* dst = cu + ((b * 8 + i) * cstep + pair * pair_bytes) + coff;
                Raw c{};
                if constexpr (!STORE) c = old[k % DEPTH][i];
                if constexpr (OUT_BF16) {
                    const u32x2 o = {pack_bf16x2_hw(v.x + bf16_lo(c[0]), v.y + bf16_hi(c[0])),
                                     pack_bf16x2_hw(v.z + bf16_lo(c[1]), v.w + bf16_hi(c[1]))};
                    __builtin_nontemporal_store(o, reinterpret_cast<u32x2*>(dst));
                } else {
                    const f32x4 o = {c[0] + v.x, c[1] + v.y, c[2] + v.z, c[3] + v.w};
                    __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(dst));
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!STORE && k + DEPTH < 8) {
            fetch_old(std::integral_constant<int, (k + DEPTH < 8) ? k + DEPTH : 0>{});
            __builtin_amdgcn_sched_barrier(0);
        }
    });
}

// The kernel is persistent: workgroup w walks tiles w, w + grid, w + 2*grid, ... of the XCD-aware
// order, and the copy stream simply runs on into the next tile, so only a workgroup's very first
// K-tiles pay memory latency.  A tile's first MFMAs take a zero C operand (no accumulator clearing),
// its scale factors are fetched under its last MFMAs, and its drain runs while the next tile's first
// two K-tiles land.
// MX: the term-split form of GemmArgs::b_k_period.  The copy stream's position in B wraps at the period, and each
// K-tile's MFMAs take a power-of-two scale 2^(-4 term) on the activation side (E8M0 byte 127 - 4 term in
// v_mfma_scale_f32_32x32x64_f8f6f4; 127 = 2^0 on the weight side), so the terms add up in the accumulator with
// their weights and nothing else changes.  b_k_period is a multiple of BK.  This form takes no row index (the
// rows of a tile follow from its position), which frees the registers the scale needs.
template <int FMT, int EPI, int SCALE, int MX = 0>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void k_gemm_nt_ring(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    constexpr bool GATE = EPI == EPI_SILU_GATE;
    constexpr int OUT_BN = GATE ? BN / 2 : BN;
    // the LDS-staged drain covers these epilogues; the launcher sends such a call here only when N is a multiple
    // of the tile's output width and C and the channel descales allow 16-byte accesses
    constexpr bool ACCUM = EPI == EPI_ACCUM_F32 || EPI == EPI_ACCUM_BF16 || EPI == EPI_STORE_F32;
    constexpr bool DRAIN = EPI == EPI_NONE || EPI == EPI_BIAS || EPI == EPI_SILU_GATE || ACCUM;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    // This workgroup's walk: workgroups go to the 8 XCDs round-robin, so with a grid that is a multiple of 8 XCD x
    // takes the contiguous range [x * per, x * per + per) of the walk order and its workgroups stride through it
    // together: what runs on an XCD at one time is 32 consecutive tiles.
    const int total_tiles = (p.tile_map ? p.tile_map[0] : p.tiles_m) * p.tiles_n;
    int my_tiles, lin0, lstep;
    if (gridDim.x % kXcds == 0) {
        const int per = (total_tiles + kXcds - 1) / kXcds;
        const int x = blockIdx.x % kXcds, i = blockIdx.x / kXcds;
        lstep = gridDim.x / kXcds;
        const int cnt = max(0, min(per, total_tiles - x * per));
        my_tiles = (cnt - i + lstep - 1) / lstep;
        lin0 = x * per + i;
    } else {
        lstep = gridDim.x;
        my_tiles = (total_tiles - static_cast<int>(blockIdx.x) + lstep - 1) / lstep;
        lin0 = blockIdx.x;
    }
    if (my_tiles <= 0) return;        // grouped launches size the grid by an upper bound of the tile count
    const int ktiles = p.K / BK;      // >= 2, checked by the launcher
    const int term_ktiles = MX ? p.b_k_period / BK : ktiles;      // K-tiles per term
    // one register for both scale operands: byte 0 = 127 (2^0, the weight side), byte 1 = 127 - 4 term (the activation side)
    constexpr int kMxOne = 0x7f7f, kMxStep = 0x0400;
    int mx_scale = kMxOne, mx_left = term_ktiles;                  // scale of the K-tile being computed
    auto mx_next = [&]() {                                         // ... moves on to the next K-tile of the tile
        if constexpr (MX) {
            if (--mx_left == 0) { mx_left = term_ktiles; mx_scale -= kMxStep; }
        }
    };

    float s1 = 0.0f, s2 = 0.0f;
    if constexpr (SCALE == SCALE_TENSOR && DRAIN) {
        s1 = p.sa[0] * p.sb[0];
        if constexpr (GATE) s2 = p.sa[0] * p.sb2[0];
    }
    if constexpr (SCALE == SCALE_ROW) s1 = p.sb[0];

    // ---- global -> LDS: wave w copies rows [64w, 64w+64) of an operand tile, 8 rows per instruction ----
    const int lrow = lane >> 3, lslot = lane & 7;
    uint32_t xoff[8], woff[8];                         // per-lane byte offsets from the operand bases
    const uint8_t* wb = p.B;                           // weight bases of the tile the copy stream is aimed at
    const uint8_t* wb2 = p.B2;
    // Where a tile lives and, for the grouped form, which A rows its 256 rows gather: everything `aim` needs
    // from memory.  Both are fetched ahead of the turn of the copy stream at points where waiting for them
    // cannot stall the copy pipeline: the position under the last K-tile of the tile two before (consumed
    // after that tile's drain has waited for all memory traffic), the rows inside that drain.
    auto fetch_pos = [&](int seq, TilePos& t) { t = locate_tile<OUT_BN>(p, lin0 + seq * lstep); };
    auto fetch_rows = [&](const TilePos& t, int (&rows)[8]) {
        if constexpr (MX) return;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int arow = min(t.m0 + wave * 64 + j * 8 + lrow, t.m_end - 1);
            rows[j] = p.a_row_index ? p.a_row_index[arow] : arow;
        }
    };
    auto fetch_tile = [&](int seq, TilePos& t, int (&rows)[8]) {
        fetch_pos(seq, t);
        fetch_rows(t, rows);
    };
    auto aim = [&](const TilePos& t, const int (&rows)[8]) {      // point the copy stream at a fetched tile
        wb = p.B + t.expert * p.b_expert_stride;
        if constexpr (GATE) wb2 = p.B2 + t.expert * p.b_expert_stride;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = wave * 64 + j * 8 + lrow;
            const uint32_t gchunk = (lslot ^ swz(row)) * 16;
            const int arow = MX ? min(t.m0 + row, t.m_end - 1) : rows[j];
            xoff[j] = static_cast<uint32_t>(arow) * static_cast<uint32_t>(p.lda) + gchunk;
            int n = t.n0 + row;
            if constexpr (GATE) {
                // LDS weight rows of a wave: [gate 32 | up 32 | gate 32 | up 32] over the same 64 output columns;
                // copies j < 4 of a wave read the gate matrix, j >= 4 the up matrix
                n = t.n0 + (row >> 7) * 64 + ((row >> 6) & 1) * 32 + (row & 31);
            }
            woff[j] = static_cast<uint32_t>(min(n, p.N - 1)) * static_cast<uint32_t>(p.ldb) + gchunk;
        }
    };
    // The copies are issued through inline assembly: the compiler cannot tell that an LDS-DMA write
    // and a later LDS read touch different slots, and would wait for every outstanding copy before
    // each operand read.  Their completion is tracked by hand with s_waitcnt vmcnt before the barriers.
    uint32_t lds_wave = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)) + wave * (64 * BK);
    // copy instruction J (0..7) of an operand tile into the ring slot at byte offset `slot`
    auto dma = [&](int slot, uint32_t voff, const uint8_t* base, auto jc) {
        constexpr int J = decltype(jc)::value;
        const uint32_t dst = lds_wave + slot;
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     :: "s"(dst), "n"(J * 8 * BK), "v"(voff), "s"(base) : "memory", "scc");
    };
    auto dma_x = [&](int slot, int k0, auto jc) { dma(slot, xoff[decltype(jc)::value], p.A + k0, jc); };
    auto dma_w = [&](int slot, int k0, auto jc) {
        constexpr int J = decltype(jc)::value;
        dma(slot, woff[J], ((GATE && J >= 4) ? wb2 : wb) + k0, jc);
    };

    // ---- LDS -> MFMA operands ----
    const int frow = lane & 31, khalf = lane >> 5, fs = swz(frow);
    int rd[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 2; ++j) rd[h][j] = frow * BK + (((h * 4 + khalf * 2 + j) ^ fs) << 4);
    const uint8_t* xrd = smem + wm * 128 * BK;
    const uint8_t* wrd = smem + wn * 128 * BK;

    v16f acc[4][4];
    // operand registers, two sets: k-half h of any K-tile lives in set h
    v8i wq[2][4], xq[2][4];
    auto put = [](v8i& dst, int half, const uint4 v) {
        dst[4 * half + 0] = (int)v.x; dst[4 * half + 1] = (int)v.y; dst[4 * half + 2] = (int)v.z; dst[4 * half + 3] = (int)v.w;
    };
    // read I (0..15) of k-half H from the X tile in slot sx and the W tile in slot sw, in the order the
    // MFMAs need them: w0 x0 x1 x2 x3 w1 w2 w3, two reads each
    auto read_one = [&](int sx, int sw, auto hc, auto ic) {
        constexpr int H = decltype(hc)::value, I = decltype(ic)::value;
        constexpr int t = I >> 1, half = I & 1;
        const int r = rd[H][half];
        if constexpr (t == 0)      put(wq[H][0], half, *reinterpret_cast<const uint4*>(wrd + sw + r));
        else if constexpr (t <= 4) put(xq[H][t - 1], half, *reinterpret_cast<const uint4*>(xrd + sx + (t - 1) * 32 * BK + r));
        else                       put(wq[H][t - 4], half, *reinterpret_cast<const uint4*>(wrd + sw + (t - 4) * 32 * BK + r));
    };
    auto mfma_one = [&](auto hc, auto ic, auto first_c) {
        constexpr int H = decltype(hc)::value, I = decltype(ic)::value;
        constexpr int a = I >> 2, b = I & 3;
        v16f c = acc[a][b];
        if constexpr (decltype(first_c)::value != 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) c[r] = 0.0f;
        }
        if constexpr (MX)
            acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wq[H][a], xq[H][b], c, (FMT >> 1) & 1, FMT & 1, 0, mx_scale, 1, mx_scale);
        else
            acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wq[H][a], xq[H][b], c, (FMT >> 1) & 1, FMT & 1, 0, 0, 0, 0);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;

    // ring slots (byte offsets) of the operand tiles around the current K-tile g:
    // a0 = X(g), a1 = W(g), a2 = X(g+1), a3 = W(g+1), a4 = the slot X(g+2) is copied into; W(g+2) goes into a0
    int a0 = 0, a1 = kSlotBytes, a2 = 2 * kSlotBytes, a3 = 3 * kSlotBytes, a4 = 4 * kSlotBytes;

    TileScales<EPI> sc;

    // One K-tile g: X(g+2) and W(g+2) are started, K-tile g+1 is waited for (unless `wait` is false: then it
    // is known to have landed) and made visible by the barrier.  FIRST: the tile's first K-tile (zero C
    // operand).  END: the tile's last K-tile: the operands of the next tile are read after the drain, and
    // the drain's first scale factors are fetched here instead.
    // tiles of this workgroup around the one being computed: t0 = current, t1 = next, t2 = the one after;
    // nrows = the A rows of the tile the copy stream turns to next
    TilePos t0, t1, t2;
    int nrows[8];
    int fetch_seq = 0;                                 // the tile END fetches next (into t2 / nrows)

    auto ktile = [&](auto first_c, auto end_c, int dk0, int dkw, const TilePos& t, bool wait) {
        constexpr bool END = decltype(end_c)::value != 0;
        // step (g,0)
        static_for<0, 16>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            mfma_one(C0{}, ic, first_c);
            read_one(a0, a1, C1{}, ic);
            if constexpr (i >= 2 && i < 10) dma_x(a4, dk0, std::integral_constant<int, (i >= 2 && i < 10) ? i - 2 : 0>{});
            __builtin_amdgcn_sched_barrier(0);
        });
        // step (g,1)
        mfma_one(C1{}, C0{}, C0{});
        mfma_one(C1{}, C1{}, C0{});
        __builtin_amdgcn_sched_barrier(0);
        if (wait) __builtin_amdgcn_s_waitcnt(kWaitVm8);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        static_for<2, 16>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            mfma_one(C1{}, ic, C0{});
            if constexpr (!END) {
                read_one(a2, a3, C0{}, std::integral_constant<int, i - 2>{});
                if constexpr (i >= 14) read_one(a2, a3, C0{}, ic);       // reads 14 and 15 ride with the last two MFMAs
            }
            if constexpr (i >= 2 && i < 10) dma_w(a0, dkw, std::integral_constant<int, (i >= 2 && i < 10) ? i - 2 : 0>{});
            if constexpr (END && i == 11) {
                if (fetch_seq < my_tiles) fetch_pos(fetch_seq, t2);
            }
            if constexpr (END && DRAIN && !ACCUM && i == 10) {
                load_row_scales<EPI, SCALE>(sc, p, t, wm, lane);
                load_pair_scales<EPI, SCALE>(sc.cs, sc.cs2, p, t, wn, lane, 0);
            }
            if constexpr (END && ACCUM && SCALE == SCALE_ROW && i == 10) load_row_scales<EPI, SCALE>(sc, p, t, wm, lane);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto rotate = [&]() {
        const int b0 = a0, b1 = a1;
        a0 = a2; a1 = a3; a2 = a4; a3 = b0; a4 = b1;
    };

    // Copy position: two K-tiles ahead of the compute position (ktiles >= 2, so at most one tile ahead).
    // Past the workgroup's last tile the stream simply re-reads that tile: the last two K-tiles then run
    // the same code as every other one, and what they copy is never used.
    int dkt = 2 % ktiles, dseq = 2 / ktiles;
    int dkw = (dkt % term_ktiles) * BK;        // the stream's position in B (bytes along K): wraps at the term length
    // With three or more K-tiles per tile the stream turns to tile s+1 while tile s is being computed, and
    // (t1, nrows) were fetched under the last K-tile of tile s-1.  With two K-tiles per tile the stream is a
    // whole tile ahead; that shape simply fetches at the turn and waits.
    const bool ahead = ktiles > 2;

    // prologue: tile 0 located and aimed at, tile 1 fetched, and all of these loads waited for before the
    // first copy is issued (the copy pipeline must never wait on them); then K-tiles 0 and 1 of the stream
    // in flight, K-tile 0 landed and visible, operands (0,0) in set 0
    {
        int rows0[8] = {};
        fetch_tile(0, t0, rows0);
        aim(t0, rows0);
        t1 = t0; t2 = t0;
#pragma unroll
        for (int j = 0; j < 8; ++j) nrows[j] = rows0[j];
        if (ahead && my_tiles > 1) fetch_tile(1, t1, nrows);
        __builtin_amdgcn_s_waitcnt(kWaitVm0);
        static_for<0, 8>([&](auto jc) { dma_x(a0, 0, jc); });
        static_for<0, 8>([&](auto jc) { dma_w(a1, 0, jc); });
        static_for<0, 8>([&](auto jc) { dma_x(a2, BK, jc); });
        static_for<0, 8>([&](auto jc) { dma_w(a3, (1 % term_ktiles) * BK, jc); });
        if (!ahead && my_tiles > 1) {
            fetch_tile(1, t1, rows0);
            aim(t1, rows0);
        }
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm16);
    __syncthreads();
    static_for<0, 16>([&](auto ic) { read_one(a0, a1, C0{}, ic); });

    auto advance_copy = [&]() {
        dkw += BK;
        if (MX && dkw == p.b_k_period) dkw = 0;
        if (++dkt == ktiles) {                   // the stream moves on to the next tile
            dkt = 0;
            dkw = 0;
            if (++dseq < my_tiles) {
                if (ahead) {
                    aim(t1, nrows);
                } else {
                    TilePos tt;
                    int rr[8] = {};
                    fetch_tile(dseq, tt, rr);
                    aim(tt, rr);
                }
            }
        }
    };

    for (int seq = 0; seq < my_tiles; ++seq) {
        if (!ahead) fetch_pos(seq, t0);
        const TilePos t = t0;
        // after a drain the first K-tile's successor has been waited for already
        if constexpr (MX) { mx_scale = kMxOne; mx_left = term_ktiles; }
        ktile(C1{}, C0{}, dkt * BK, dkw, t, !(DRAIN && seq > 0));
        rotate(); advance_copy(); mx_next();
        for (int kt = 1; kt + 1 < ktiles; ++kt) {
            ktile(C0{}, C0{}, dkt * BK, dkw, t, true);
            rotate(); advance_copy(); mx_next();
        }
        fetch_seq = ahead ? seq + 2 : my_tiles;       // what the last K-tile fetches into (t2, nrows)
        ktile(C0{}, C1{}, dkt * BK, dkw, t, true);
        rotate(); advance_copy();
        // After the rotation a4 is the slot that held W of the K-tile just finished.  Every wavefront has
        // finished reading it (barrier of the last step) and only X of the stream's third K-tile from here
        // is copied into it next, by this wavefront's own copies, in program order after the drain.
        // the rows of the tile fetched under the last K-tile: loaded inside the drain, right after its wait
        const bool more = ahead && seq + 2 < my_tiles;
        auto landed = [&]() { if (more) fetch_rows(t2, nrows); };
        if constexpr (DRAIN) {
            uint8_t* stage = smem + a4 + wave * (64 * BK);
            if constexpr (ACCUM) {
                constexpr bool BF = EPI == EPI_ACCUM_BF16, ST = EPI == EPI_STORE_F32;
                if constexpr (SCALE != SCALE_ROW) {
#pragma unroll
                    for (int b = 0; b < 4; ++b) sc.sa[b] = 1.0f;
                }
                if (t.m0 + BM <= t.m_end && t.n0 + BN <= p.N) drain_tile_accum<false, BF, ST>(acc, sc.sa, s1, p, t, wm, wn, lane, stage, landed);
                else                      drain_tile_accum<true, BF, ST>(acc, sc.sa, s1, p, t, wm, wn, lane, stage, landed);
            } else {
                constexpr int out_bn = EPI == EPI_SILU_GATE ? BN / 2 : BN;
                if (t.m0 + BM <= t.m_end && t.n0 + out_bn <= p.N) drain_tile<EPI, SCALE, false>(acc, sc, s1, s2, p, t, wm, wn, lane, stage, landed);
                else                      drain_tile<EPI, SCALE, true>(acc, sc, s1, s2, p, t, wm, wn, lane, stage, landed);
            }
        } else {
            landed();
            GemmArgs q = p;                        // the epilogue sees this tile's row bound
            q.M = t.m_end;
            epilogue<EPI, SCALE>(acc, q, t.m0, t.n0, wm, wn, lane);
        }
        if (more && !MX) {
            // the row loads are older than the drain's last stores: requiring them here waits for nothing else
#pragma unroll
            for (int j = 0; j < 8; ++j) asm volatile("" :: "v"(nrows[j]));
        }
        t0 = t1; t1 = t2;
        static_for<0, 16>([&](auto ic) { read_one(a0, a1, C0{}, ic); });
    }
    // the copies started past the end of the stream must have landed before the LDS is given back
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
}

// ---- ring kernel on the 16 x 16 x 128 MFMA -----------------------------------------------------------------
// The same persistent structure, ring, copy stream, tile walk and drain staging as k_gemm_nt_ring, with the
// products taken by v_mfma_f32_16x16x128_f8f6f4 instead of v_mfma_f32_32x32x64_f8f6f4.  Both shapes do 2048 FLOP
// per cycle and SIMD; measured on this part, MFMAs alone on random E4M3 operands, the 16 x 16 x 128 shape delivers
// 8 - 9 % more at the same socket power (and draws 10 % less on constant operands), and these GEMMs run at the power
// cap.  A wavefront's 128 x 128 tile is 8 x 8 blocks of 16 x 16 (four accumulator registers each, 256 in all); an
// MFMA consumes a whole 128-byte K-tile row of both operands, so every accumulator is touched once per K-tile.
// Operand registers: four sets of four blocks (weights: N-halves A0, A1; activations: M-halves B0, B1; 32 registers
// each).  A K-tile is four phases of sixteen MFMAs; with parity p of the K-tile they use
//   (A0, B[p]) -> (A0, B[1-p]) -> (A1, B[1-p]) -> (A1, B[p])
// and the set that a phase has left behind is refilled two phases before it is needed again: B[1-p] and A1 of this
// K-tile under phases 0 and 1, A0 and B[1-p] of the NEXT K-tile under phases 2 and 3 (after the barrier that makes
// that K-tile visible).  The next K-tile then starts with (A0, B[1-p]): its parity is the other one, and so on.
// Forms: plain, bias and SiLU-gate epilogues (the LDS-staged bf16 drain), every scale mode of those, dense or
// grouped, an even number of K-tiles.  The accumulate / fp32-store forms stay on k_gemm_nt_ring (the fp32-accumulating
// weight gradient measured the same on either shape: its drain, not the MFMAs, sets its power), and so does the
// term-split form.
typedef float v4f __attribute__((ext_vector_type(4)));
// 16-byte chunk swizzle of this kernel's operand tiles: within any 16 rows the 16-lane groups of a ds_read_b128 (rows
// 0-7 of one k-group with rows 8-15 of the next) land in 16 different 16-byte slots of a 256-byte line, and the
// pattern repeats every 16 rows
__device__ __forceinline__ int swz16(int row) { return (row ^ ((row >> 3) & 1)) & 7; }

template <int EPI>
struct TileScales16 {
    float sa[8];           // descales of this lane's eight output rows (row j * 16 + lane % 16 of the wavefront's 128)
    float4 cs[2][2];       // channel descales of the pair being drained: [unit in pair][16-column block], this lane's 4 columns
    float4 cs2[2][2];      // up-projection descales (SiLU-gate)
};

template <int EPI, int SCALE>
__device__ __forceinline__ void load_row_scales16(TileScales16<EPI>& s, const GemmArgs& p, const TilePos& t, int wm, int lane) {
    if constexpr (SCALE == SCALE_ROWCOL || SCALE == SCALE_ROW) {
        int r[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = min(t.m0 + wm * 128 + j * 16 + (lane & 15), t.m_end - 1);
        if (p.a_row_index) {
#pragma unroll
            for (int j = 0; j < 8; ++j) r[j] = p.a_row_index[r[j]];
#pragma unroll
            for (int j = 0; j < 8; ++j) s.sa[j] = p.sa[r[j]];
            asm volatile("; row scales through the row index" ::: "memory");
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) s.sa[j] = p.sa[r[j]];
        }
    }
}
template <int EPI, int SCALE>
__device__ __forceinline__ void load_pair_scales16(float4 (&cs)[2][2], float4 (&cs2)[2][2], const GemmArgs& p,
                                                   const TilePos& t, int wn, int lane, int pair) {
    constexpr int NU = EPI == EPI_SILU_GATE ? 2 : 4;
    const size_t col0 = t.n0 + wn * (NU * 32) + pair * 64;
    if constexpr (SCALE == SCALE_ROWCOL) {
        const size_t ucol = static_cast<size_t>(t.expert) * p.sb_expert_stride + col0;
        const uint8_t* b1 = reinterpret_cast<const uint8_t*>(p.sb + ucol);
        const uint8_t* b2 = reinterpret_cast<const uint8_t*>(EPI == EPI_SILU_GATE ? p.sb2 + ucol : p.sb);
        const uint32_t loff = static_cast<uint32_t>(lane >> 4) * 16u;      // this lane's four columns of a 16-column block
        if constexpr (EPI != EPI_SILU_GATE) {
            if (t.n0 + BN > p.N) {      // a last column tile that N cuts short: unused factors are read from the last four columns
                const int lim = (p.N - 4 - static_cast<int>(col0)) * 4;
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int sb = 0; sb < 2; ++sb)
                        cs[u][sb] = *reinterpret_cast<const float4*>(b1 + min(static_cast<int>(loff + u * 128u + sb * 64u), lim));
                return;
            }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int sb = 0; sb < 2; ++sb) {
                cs[u][sb] = *reinterpret_cast<const float4*>(b1 + (loff + u * 128u + sb * 64u));
                if constexpr (EPI == EPI_SILU_GATE) cs2[u][sb] = *reinterpret_cast<const float4*>(b2 + (loff + u * 128u + sb * 64u));
            }
    }
}

// The drain of k_gemm_nt_ring for the 16 x 16 accumulator blocks: lane l of block (i, j) holds output row
// j * 16 + l % 16 and the four consecutive columns i * 16 + 4 (l / 16) ... + 3 of the wavefront's 128 accumulated
// columns.  Staging layout, read-back and stores are those of drain_tile.
template <int EPI, int SCALE, bool RAGGED, class Landed>
__device__ __forceinline__ void drain_tile16(v4f (&acc)[8][8], TileScales16<EPI>& s, float s1, float s2, const GemmArgs& p,
                                             const TilePos& t, int wm, int wn, int lane, uint8_t* stage, Landed&& landed) {
    constexpr bool GATE = EPI == EPI_SILU_GATE;
    constexpr int NU = GATE ? 2 : 4;
    const int row16 = lane & 15, cq = lane >> 4;
    const int rr = lane >> 3, rc = lane & 7;
    const uint8_t* rdp0 = stage + rr * 128 + ((rc ^ (rr >> 1)) << 4);
    const uint8_t* rdp1 = stage + rr * 128 + ((rc ^ (rr >> 1) ^ 4) << 4);
    const int mrow0 = t.m0 + wm * 128 + rr;
    uint8_t* cu = reinterpret_cast<uint8_t*>(p.C + static_cast<size_t>(t.m0 + wm * 128) * p.ldc + t.n0 + wn * (NU * 32));
    const uint32_t coff = (static_cast<uint32_t>(rr) * static_cast<uint32_t>(p.ldc) + rc * 8u) * 2u;
    const size_t cstep = static_cast<size_t>(p.ldc) * 16;
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    uint4 bias8[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
    if constexpr (EPI == EPI_BIAS) {
        const int bcol = t.n0 + wn * (NU * 32) + rc * 8;
#pragma unroll
        for (int pair = 0; pair < NU / 2; ++pair)
            bias8[pair] = *reinterpret_cast<const uint4*>(p.bias + (RAGGED ? min(bcol + pair * 64, p.N - 8) : bcol + pair * 64));
    }
    const int ncol0 = t.n0 + wn * (NU * 32) + rc * 8;

#pragma unroll
    for (int pair = 0; pair < NU / 2; ++pair) {
        const uint4 bv = bias8[pair];
        const float bf[8] = {bf16_lo(bv.x), bf16_hi(bv.x), bf16_lo(bv.y), bf16_hi(bv.y),
                             bf16_lo(bv.z), bf16_hi(bv.z), bf16_lo(bv.w), bf16_hi(bv.w)};
        float4 ncs[2][2], ncs2[2][2];
        if (pair + 1 < NU / 2) load_pair_scales16<EPI, SCALE>(ncs, ncs2, p, t, wn, lane, pair + 1);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int j = half * 4 + jj;
                const float sa = (SCALE == SCALE_ROWCOL || SCALE == SCALE_ROW) ? s.sa[j] : 1.0f;
                const int R = jj * 16 + row16;                       // row of the 64-row staging block
                uint8_t* wr = stage + R * 128 + (cq & 1) * 8;
                const int wswz = (R >> 1) & 7;
#pragma unroll
                for (int u = 0; u < 2; ++u) {
#pragma unroll
                    for (int sb = 0; sb < 2; ++sb) {
                        float4 c = make_float4(s1, s1, s1, s1), up = make_float4(s2, s2, s2, s2);
                        if constexpr (SCALE == SCALE_ROWCOL) {
                            c = s.cs[u][sb];
                            if constexpr (GATE) up = s.cs2[u][sb];
                        }
                        const float c4[4] = {c.x, c.y, c.z, c.w}, u4[4] = {up.x, up.y, up.z, up.w};
                        float v[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            if constexpr (GATE) {
                                // weight rows of the wavefront: [gate 32 | up 32 | gate 32 | up 32]: unit u = blocks 4u .. 4u + 3
                                const uint32_t gu = pack_bf16x2_hw(acc_read(acc[u * 4 + sb][j][q]) * (sa * c4[q]),
                                                                   acc_read(acc[u * 4 + 2 + sb][j][q]) * (sa * u4[q]));
                                v[q] = fast_silu(bf16_lo(gu)) * bf16_hi(gu);
                            } else {
                                v[q] = acc_read(acc[pair * 4 + u * 2 + sb][j][q]) * (sa * c4[q]);
                            }
                        }
                        *reinterpret_cast<uint2*>(wr + (((u * 4 + sb * 2 + (cq >> 1)) ^ wswz) << 4)) =
                            make_uint2(pack_bf16x2_hw(v[0], v[1]), pack_bf16x2_hw(v[2], v[3]));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (pair == 0 && half == 0) {
                __builtin_amdgcn_s_waitcnt(kWaitVm0);
                landed();
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint4 v = *reinterpret_cast<const uint4*>(((i & 1) ? rdp1 : rdp0) + i * 8 * 128);
                if constexpr (EPI == EPI_BIAS) {
                    v.x = pack_bf16x2_hw(bf16_lo(v.x) + bf[0], bf16_hi(v.x) + bf[1]);
                    v.y = pack_bf16x2_hw(bf16_lo(v.y) + bf[2], bf16_hi(v.y) + bf[3]);
                    v.z = pack_bf16x2_hw(bf16_lo(v.z) + bf[4], bf16_hi(v.z) + bf[5]);
                    v.w = pack_bf16x2_hw(bf16_lo(v.w) + bf[6], bf16_hi(v.w) + bf[7]);
                }
                if (!RAGGED || (mrow0 + half * 64 + i * 8 < t.m_end && ncol0 + pair * 64 < p.N)) {
                    const u32x4 vv = {v.x, v.y, v.z, v.w};
                    __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>(cu + ((half * 8 + i) * cstep + pair * 128) + coff));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (pair + 1 < NU / 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int sb = 0; sb < 2; ++sb) { s.cs[u][sb] = ncs[u][sb]; s.cs2[u][sb] = ncs2[u][sb]; }
        }
    }
}

// A K-tile's parity is its position in the tile modulo 2 (after a drain the operands are read afresh, so every tile
// starts at parity 0).  The number of K-tiles per tile is even (the launcher sends other shapes to k_gemm_nt_ring), so a
// tile is first(0), pairs of (1, 0), last(1): straight-line code.  (Two forms for odd counts were built and measured at
// K = 1408 against k_gemm_nt_ring: first(0), pairs of (1, 0), 1, last(0) spilled registers inside the K-tile loop and ran
// 20 % slower; first(0), 1, pairs of (0, 1), last(0) ran 1 % slower.  Eleven K-tiles per drain leave the matrix cores too
// little of the launch for their lower power to pay.)
template <int FMT, int EPI, int SCALE>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
void k_gemm_nt_ring16(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    static_assert(EPI == EPI_NONE || EPI == EPI_BIAS || EPI == EPI_SILU_GATE, "bf16 drain forms only");
    constexpr bool GATE = EPI == EPI_SILU_GATE;
    constexpr int OUT_BN = GATE ? BN / 2 : BN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int total_tiles = (p.tile_map ? p.tile_map[0] : p.tiles_m) * p.tiles_n;
    int my_tiles, lin0, lstep;
    if (gridDim.x % kXcds == 0) {
        const int per = (total_tiles + kXcds - 1) / kXcds;
        const int x = blockIdx.x % kXcds, i = blockIdx.x / kXcds;
        lstep = gridDim.x / kXcds;
        const int cnt = max(0, min(per, total_tiles - x * per));
        my_tiles = (cnt - i + lstep - 1) / lstep;
        lin0 = x * per + i;
    } else {
        lstep = gridDim.x;
        my_tiles = (total_tiles - static_cast<int>(blockIdx.x) + lstep - 1) / lstep;
        lin0 = blockIdx.x;
    }
    if (my_tiles <= 0) return;
    const int ktiles = p.K / BK;      // >= 2, checked by the launcher

    float s1 = 0.0f, s2 = 0.0f;
    if constexpr (SCALE == SCALE_TENSOR) {
        s1 = p.sa[0] * p.sb[0];
        if constexpr (GATE) s2 = p.sa[0] * p.sb2[0];
    }
    if constexpr (SCALE == SCALE_ROW) s1 = p.sb[0];

    // ---- global -> LDS: as in k_gemm_nt_ring ----
    const int lrow = lane >> 3, lslot = lane & 7;
    uint32_t xoff[8], woff[8];
    const uint8_t* wb = p.B;
    const uint8_t* wb2 = p.B2;
    auto fetch_pos = [&](int seq, TilePos& t) { t = locate_tile<OUT_BN>(p, lin0 + seq * lstep); };
    auto fetch_rows = [&](const TilePos& t, int (&rows)[8]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int arow = min(t.m0 + wave * 64 + j * 8 + lrow, t.m_end - 1);
            rows[j] = p.a_row_index ? p.a_row_index[arow] : arow;
        }
    };
    auto fetch_tile = [&](int seq, TilePos& t, int (&rows)[8]) {
        fetch_pos(seq, t);
        fetch_rows(t, rows);
    };
    auto aim = [&](const TilePos& t, const int (&rows)[8]) {
        wb = p.B + t.expert * p.b_expert_stride;
        if constexpr (GATE) wb2 = p.B2 + t.expert * p.b_expert_stride;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = wave * 64 + j * 8 + lrow;
            const uint32_t gchunk = (lslot ^ swz16(row)) * 16;
            xoff[j] = static_cast<uint32_t>(rows[j]) * static_cast<uint32_t>(p.lda) + gchunk;
            int n = t.n0 + row;
            if constexpr (GATE) n = t.n0 + (row >> 7) * 64 + ((row >> 6) & 1) * 32 + (row & 31);
            woff[j] = static_cast<uint32_t>(min(n, p.N - 1)) * static_cast<uint32_t>(p.ldb) + gchunk;
        }
    };
    uint32_t lds_wave = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)) + wave * (64 * BK);
    auto dma = [&](int slot, uint32_t voff, const uint8_t* base, auto jc) {
        constexpr int J = decltype(jc)::value;
        // (the slot offsets rotate through five variables; the compiler may park one in a vector register)
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_wave + slot);
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     :: "s"(dst), "n"(J * 8 * BK), "v"(voff), "s"(base) : "memory", "scc");
    };
    auto dma_x = [&](int slot, int k0, auto jc) { dma(slot, xoff[decltype(jc)::value], p.A + k0, jc); };
    auto dma_w = [&](int slot, int k0, auto jc) {
        constexpr int J = decltype(jc)::value;
        dma(slot, woff[J], ((GATE && J >= 4) ? wb2 : wb) + k0, jc);
    };

    // ---- LDS -> MFMA operands: block b of an operand half is rows b * 16 ... + 15; lane l reads row l % 16, the
    // 32 bytes of k-group l / 16 (two swizzled 16-byte chunks).  The swizzle is the same for every block, so a set's
    // eight reads are two addresses plus immediates. ----
    const int r16 = lane & 15, kg = lane >> 4;
    int rd[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) rd[c] = r16 * BK + (((kg * 2 + c) ^ swz16(r16)) << 4);
    const uint8_t* xrd = smem + wm * 128 * BK;
    const uint8_t* wrd = smem + wn * 128 * BK;

    v4f acc[8][8];
    v8i WA[2][4], XB[2][4];       // operand sets: weights N-halves, activations M-halves
    auto put = [](v8i& dst, int half, const uint4 v) {
        dst[4 * half + 0] = (int)v.x; dst[4 * half + 1] = (int)v.y; dst[4 * half + 2] = (int)v.z; dst[4 * half + 3] = (int)v.w;
    };
    // read R (0..7) of a set: block R / 2, chunk R % 2.  SET: 0, 1 = weights A0, A1 from slot `slot`; 2, 3 = activations B0, B1
    auto read_set = [&](int slot, auto setc, auto rc_) {
        constexpr int SET = decltype(setc)::value, R = decltype(rc_)::value;
        constexpr int blk = R >> 1, c = R & 1;
        constexpr int gb = (SET & 1) * 4 + blk;              // block within the wavefront's 128 rows
        const int off = slot + gb * 16 * BK + rd[c];
        if constexpr (SET < 2) put(WA[SET][blk], c, *reinterpret_cast<const uint4*>(wrd + off));
        else                   put(XB[SET - 2][blk], c, *reinterpret_cast<const uint4*>(xrd + off));
    };
    auto mfma_blk = [&](auto sac, auto sbc, auto ic, auto first_c) {
        constexpr int SA = decltype(sac)::value, SB = decltype(sbc)::value, I = decltype(ic)::value;
        constexpr int ii = I >> 2, jj = I & 3;
        v4f c = acc[SA * 4 + ii][SB * 4 + jj];
        if constexpr (decltype(first_c)::value != 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) c[r] = 0.0f;
        }
        acc[SA * 4 + ii][SB * 4 + jj] =
            __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(WA[SA][ii], XB[SB][jj], c, (FMT >> 1) & 1, FMT & 1, 0, 0, 0, 0);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;

    int a0 = 0, a1 = kSlotBytes, a2 = 2 * kSlotBytes, a3 = 3 * kSlotBytes, a4 = 4 * kSlotBytes;
    TileScales16<EPI> sc;
    TilePos t0, t1, t2;
    int nrows[8];
    int fetch_seq = 0;

    // One K-tile g of parity P.  Phases 0 and 1 (32 MFMAs): the X copies of K-tile g+2 into a4, the reads of B[1-P]
    // and A1 of this K-tile; wait + barrier; phases 2 and 3: the W copies of K-tile g+2 into a0, the reads of A0 and
    // B[1-P] of K-tile g+1 (not in a tile's last K-tile: the next tile's operands are read after the drain).
    auto ktile = [&](auto first_c, auto end_c, auto par_c, int dk0, const TilePos& t, bool wait) {
        constexpr bool END = decltype(end_c)::value != 0;
        constexpr int P = decltype(par_c)::value;
        using SBP = std::integral_constant<int, P>;             // activations set of phases 0 and 3
        using SBQ = std::integral_constant<int, 1 - P>;         // ... of phases 1 and 2
        using RBQ = std::integral_constant<int, 2 + (1 - P)>;   // read_set index of B[1-P]
        static_for<0, 16>([&](auto ic) {                        // phase 0: (A0, B[P]); reads B[1-P](g)
            constexpr int i = decltype(ic)::value;
            mfma_blk(C0{}, SBP{}, ic, first_c);
            if constexpr ((i & 1) == 0) read_set(a0, RBQ{}, std::integral_constant<int, i / 2>{});
            if constexpr (i >= 4 && (i & 1) == 1) dma_x(a4, dk0, std::integral_constant<int, (i >= 4) ? (i - 5) / 2 : 0>{});
            __builtin_amdgcn_sched_barrier(0);
        });
        static_for<0, 16>([&](auto ic) {                        // phase 1: (A0, B[1-P]); reads A1(g)
            constexpr int i = decltype(ic)::value;
            mfma_blk(C0{}, SBQ{}, ic, first_c);
            if constexpr ((i & 1) == 0) read_set(a1, C1{}, std::integral_constant<int, i / 2>{});
            if constexpr (i < 4 && (i & 1) == 1) dma_x(a4, dk0, std::integral_constant<int, 6 + i / 2>{});
            __builtin_amdgcn_sched_barrier(0);
        });
        // phase 2: (A1, B[1-P])
        mfma_blk(C1{}, SBQ{}, C0{}, first_c);
        mfma_blk(C1{}, SBQ{}, C1{}, first_c);
        __builtin_amdgcn_sched_barrier(0);
        if (wait) __builtin_amdgcn_s_waitcnt(kWaitVm8);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        static_for<2, 16>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            mfma_blk(C1{}, SBQ{}, ic, first_c);
            if constexpr (!END && (i & 1) == 0) read_set(a3, C0{}, std::integral_constant<int, (i - 2) / 2>{});      // A0(g+1): reads 0..6
            if constexpr ((i & 1) == 1) dma_w(a0, dk0, std::integral_constant<int, (i - 3) / 2>{});                  // W copies 0..6
            __builtin_amdgcn_sched_barrier(0);
        });
        static_for<0, 16>([&](auto ic) {                        // phase 3: (A1, B[P]); reads B[1-P](g+1)
            constexpr int i = decltype(ic)::value;
            mfma_blk(C1{}, SBP{}, ic, first_c);
            if constexpr (!END && i == 0) read_set(a3, C0{}, std::integral_constant<int, 7>{});
            if constexpr (i == 1) dma_w(a0, dk0, std::integral_constant<int, 7>{});
            if constexpr (!END && i >= 2 && (i & 1) == 0) read_set(a2, RBQ{}, std::integral_constant<int, (i >= 2) ? (i - 2) / 2 : 0>{});   // reads 0..6
            if constexpr (!END && i == 15) read_set(a2, RBQ{}, std::integral_constant<int, 7>{});
            if constexpr (END && i == 5) {
                if (fetch_seq < my_tiles) fetch_pos(fetch_seq, t2);
            }
            if constexpr (END && i == 3) {
                load_row_scales16<EPI, SCALE>(sc, p, t, wm, lane);
                load_pair_scales16<EPI, SCALE>(sc.cs, sc.cs2, p, t, wn, lane, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto rotate = [&]() {
        const int b0 = a0, b1 = a1;
        a0 = a2; a1 = a3; a2 = a4; a3 = b0; a4 = b1;
    };

    int dkt = 2 % ktiles, dseq = 2 / ktiles;
    const bool ahead = ktiles > 2;
    {
        int rows0[8] = {};
        fetch_tile(0, t0, rows0);
        aim(t0, rows0);
        t1 = t0; t2 = t0;
#pragma unroll
        for (int j = 0; j < 8; ++j) nrows[j] = rows0[j];
        if (ahead && my_tiles > 1) fetch_tile(1, t1, nrows);
        __builtin_amdgcn_s_waitcnt(kWaitVm0);
        static_for<0, 8>([&](auto jc) { dma_x(a0, 0, jc); });
        static_for<0, 8>([&](auto jc) { dma_w(a1, 0, jc); });
        static_for<0, 8>([&](auto jc) { dma_x(a2, BK, jc); });
        static_for<0, 8>([&](auto jc) { dma_w(a3, BK, jc); });
        if (!ahead && my_tiles > 1) {
            fetch_tile(1, t1, rows0);
            aim(t1, rows0);
        }
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm16);
    __syncthreads();
    // a tile's first K-tile has parity 0: it starts with (A0, B0)
    static_for<0, 8>([&](auto rc_) { read_set(a1, C0{}, rc_); });
    static_for<0, 8>([&](auto rc_) { read_set(a0, std::integral_constant<int, 2>{}, rc_); });

    auto advance_copy = [&]() {
        if (++dkt == ktiles) {
            dkt = 0;
            if (++dseq < my_tiles) {
                if (ahead) {
                    aim(t1, nrows);
                } else {
                    TilePos tt;
                    int rr[8] = {};
                    fetch_tile(dseq, tt, rr);
                    aim(tt, rr);
                }
            }
        }
    };

    for (int seq = 0; seq < my_tiles; ++seq) {
        if (!ahead) fetch_pos(seq, t0);
        const TilePos t = t0;
        ktile(C1{}, C0{}, C0{}, dkt * BK, t, !(seq > 0));
        rotate(); advance_copy();
        for (int kt = 1; kt + 2 < ktiles; kt += 2) {
            ktile(C0{}, C0{}, C1{}, dkt * BK, t, true);
            rotate(); advance_copy();
            ktile(C0{}, C0{}, C0{}, dkt * BK, t, true);
            rotate(); advance_copy();
        }
        fetch_seq = ahead ? seq + 2 : my_tiles;
        ktile(C0{}, C1{}, C1{}, dkt * BK, t, true);
        rotate(); advance_copy();
        const bool more = ahead && seq + 2 < my_tiles;
        auto landed = [&]() { if (more) fetch_rows(t2, nrows); };
        uint8_t* stage = smem + a4 + wave * (64 * BK);
        // the drain's per-lane constants are worked out afresh for every tile: hoisted out of the tile loop they would sit
        // in registers through the K-tile loop, which has none to spare
        int lane_d = lane;
        asm volatile("" : "+v"(lane_d));
        constexpr int out_bn = EPI == EPI_SILU_GATE ? BN / 2 : BN;
        if (t.m0 + BM <= t.m_end && t.n0 + out_bn <= p.N) drain_tile16<EPI, SCALE, false>(acc, sc, s1, s2, p, t, wm, wn, lane_d, stage, landed);
        else                                              drain_tile16<EPI, SCALE, true>(acc, sc, s1, s2, p, t, wm, wn, lane_d, stage, landed);
        if (more) {
#pragma unroll
            for (int j = 0; j < 8; ++j) asm volatile("" :: "v"(nrows[j]));
        }
        t0 = t1; t1 = t2;
        static_for<0, 8>([&](auto rc_) { read_set(a1, C0{}, rc_); });
        static_for<0, 8>([&](auto rc_) { read_set(a0, std::integral_constant<int, 2>{}, rc_); });
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
}

// ---- duo kernel: the ring kernel at half the tile edge, two workgroups per CU ------------------------------
// Workgroup tile 128 x 128 x 128, four wavefronts 2 x 2, each 64 x 64 = 2 x 2 MFMA tiles (64 accumulator
// registers), the same ring of five slots at 16 KiB each: 80 KiB, so a CU holds TWO workgroups and every SIMD two
// wavefronts.  A tile's drain is vector-ALU work (scales, SiLU, bf16 rounding) during which the matrix cores of a
// one-wavefront-per-SIMD kernel idle; here the other workgroup's MFMAs run under it, provided the two are out of
// step.  The workgroup that got the upper half of the CU's LDS (readable from the hardware's LDS allocation
// register) therefore starts half a tile late.  The price is twice the LDS and L2 bytes per FLOP of the 256 x 256
// tile.  Dense and grouped per expert (128-row tiles over the 256-row tile table: an entry's second half may be
// empty), E4M3 activations and weights, per-row x per-channel scales, plain or SiLU-gate epilogue; N a multiple of
// the tile's output width.
constexpr int DM = 128;
constexpr int kDuoSlot = DM * BK;                  // 16 KiB
constexpr int kDuoLds = kSlots * kDuoSlot;         // 80 KiB
constexpr int kWaitVm4 = 0x0f74;

template <int EPI, bool STAGGER>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void k_gemm_nt_duo(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr bool GATE = EPI == EPI_SILU_GATE;
    constexpr int OUT_BN = GATE ? DM / 2 : DM;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int total_tiles = p.tiles_m * p.tiles_n;
    int my_tiles, lin0, lstep;
    if (gridDim.x % kXcds == 0) {
        const int per = (total_tiles + kXcds - 1) / kXcds;
        const int x = blockIdx.x % kXcds, i = blockIdx.x / kXcds;
        lstep = gridDim.x / kXcds;
        const int cnt = max(0, min(per, total_tiles - x * per));
        my_tiles = (cnt - i + lstep - 1) / lstep;
        lin0 = x * per + i;
    } else {
        lstep = gridDim.x;
        my_tiles = (total_tiles - static_cast<int>(blockIdx.x) + lstep - 1) / lstep;
        lin0 = blockIdx.x;
    }
    if (my_tiles <= 0) return;
    const int ktiles = p.K / BK;      // >= 2, checked by the launcher

    if constexpr (STAGGER) {
        // the second workgroup of a CU (its LDS starts above the first one's) waits about half a tile's MFMA time
        unsigned alloc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_LDS_ALLOC, 0, 12)" : "=s"(alloc));
        if (alloc != 0) {
            for (int i = 0; i < (ktiles + 15) / 16; ++i) __builtin_amdgcn_s_sleep(127);
        }
    }

    auto tile_at = [&](int seq, int& m0, int& n0) {
        int tm, tn;
        tile_coords(lin0 + seq * lstep, p.tiles_m, p.tiles_n, tm, tn);
        m0 = tm * DM;
        n0 = tn * OUT_BN;
    };

    // ---- global -> LDS: wave w copies rows [32w, 32w+32) of an operand tile, 8 rows per instruction ----
    const int lrow = lane >> 3, lslot = lane & 7;
    uint32_t xoff[4], woff[4];
    // SiLU-gate: the W tile's rows are [gate 32 | up 32] for the columns of wavefront column 0, then the same for
    // column 1, so wave w copies from one matrix only: gate for even w, up for odd w
    const uint8_t* wsrc = (GATE && (wave & 1)) ? p.B2 : p.B;
    auto aim = [&](int seq) {
        int m0, n0;
        tile_at(seq, m0, n0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = wave * 32 + j * 8 + lrow;
            const uint32_t gchunk = (lslot ^ swz(row)) * 16;
            xoff[j] = static_cast<uint32_t>(min(m0 + row, p.M - 1)) * static_cast<uint32_t>(p.lda) + gchunk;
            const int n = GATE ? n0 + (row >> 6) * 32 + (row & 31) : n0 + row;
            woff[j] = static_cast<uint32_t>(min(n, p.N - 1)) * static_cast<uint32_t>(p.ldb) + gchunk;
        }
    };
    uint32_t lds_wave = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)) + wave * (32 * BK);
    auto dma = [&](int slot, uint32_t voff, const uint8_t* base, auto jc) {
        constexpr int J = decltype(jc)::value;
        const uint32_t dst = lds_wave + slot;
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     :: "s"(dst), "n"(J * 8 * BK), "v"(voff), "s"(base) : "memory", "scc");
    };
    auto dma_x = [&](int slot, int k0, auto jc) { dma(slot, xoff[decltype(jc)::value], p.A + k0, jc); };
    auto dma_w = [&](int slot, int k0, auto jc) { dma(slot, woff[decltype(jc)::value], wsrc + k0, jc); };

    // ---- LDS -> MFMA operands ----
    const int frow = lane & 31, khalf = lane >> 5, fs = swz(frow);
    int rd[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 2; ++j) rd[h][j] = frow * BK + (((h * 4 + khalf * 2 + j) ^ fs) << 4);
    const uint8_t* xrd = smem + wm * 64 * BK;
    const uint8_t* wrd = smem + wn * 64 * BK;

    v16f acc[2][2];       // [weight tile][activation tile]
    v8i wq[2][2], xq[2][2];
    auto put = [](v8i& dst, int half, const uint4 v) {
        dst[4 * half + 0] = (int)v.x; dst[4 * half + 1] = (int)v.y; dst[4 * half + 2] = (int)v.z; dst[4 * half + 3] = (int)v.w;
    };
    // read I (0..7) of k-half H: w0 x0 x1 w1, two reads each
    auto read_one = [&](int sx, int sw, auto hc, auto ic) {
        constexpr int H = decltype(hc)::value, I = decltype(ic)::value;
        constexpr int t = I >> 1, half = I & 1;
        const int r = rd[H][half];
        if constexpr (t == 0)      put(wq[H][0], half, *reinterpret_cast<const uint4*>(wrd + sw + r));
        else if constexpr (t <= 2) put(xq[H][t - 1], half, *reinterpret_cast<const uint4*>(xrd + sx + (t - 1) * 32 * BK + r));
        else                       put(wq[H][1], half, *reinterpret_cast<const uint4*>(wrd + sw + 32 * BK + r));
    };
    auto mfma_one = [&](auto hc, auto ic, auto first_c) {
        constexpr int H = decltype(hc)::value, I = decltype(ic)::value;
        constexpr int a = I >> 1, b = I & 1;
        v16f c = acc[a][b];
        if constexpr (decltype(first_c)::value != 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) c[r] = 0.0f;
        }
        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wq[H][a], xq[H][b], c, 0, 0, 0, 0, 0, 0);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;

    int a0 = 0, a1 = kDuoSlot, a2 = 2 * kDuoSlot, a3 = 3 * kDuoSlot, a4 = 4 * kDuoSlot;

    // what the drain needs in registers: row descales of this lane's two output rows and the channel descales of its
    // columns (plain: cs[a][g] = four columns of quad g of weight tile a; SiLU-gate: cs[0][g] gate, cs[1][g] up)
    float sa[2];
    float4 cs[2][4];
    auto load_scales = [&](int m0, int n0) {
#pragma unroll
        for (int b = 0; b < 2; ++b) sa[b] = p.sa[min(m0 + wm * 64 + b * 32 + (lane & 31), p.M - 1)];
        if constexpr (GATE) {
            const int col = n0 + wn * 32 + khalf * 4;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                cs[0][g] = *reinterpret_cast<const float4*>(p.sb + col + g * 8);
                cs[1][g] = *reinterpret_cast<const float4*>(p.sb2 + col + g * 8);
            }
        } else {
            const int col = n0 + wn * 64 + khalf * 4;
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int g = 0; g < 4; ++g) cs[a][g] = *reinterpret_cast<const float4*>(p.sb + col + a * 32 + g * 8);
        }
    };

    auto ktile = [&](auto first_c, auto end_c, int dk0, int m0, int n0, bool wait) {
        constexpr bool END = decltype(end_c)::value != 0;
        // step (g,0): 4 MFMAs, the operand reads of (g,1), the copies of X(g+2)
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            mfma_one(C0{}, ic, first_c);
            read_one(a0, a1, C1{}, std::integral_constant<int, 2 * i>{});
            read_one(a0, a1, C1{}, std::integral_constant<int, 2 * i + 1>{});
            dma_x(a4, dk0, ic);
            __builtin_amdgcn_sched_barrier(0);
        });
        // step (g,1)
        mfma_one(C1{}, C0{}, C0{});
        __builtin_amdgcn_sched_barrier(0);
        if (wait) __builtin_amdgcn_s_waitcnt(kWaitVm4);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        static_for<1, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            mfma_one(C1{}, ic, C0{});
            if constexpr (!END) {
                static_for<0, 3>([&](auto jc) {
                    constexpr int j = (i - 1) * 3 + decltype(jc)::value;
                    if constexpr (j < 8) read_one(a2, a3, C0{}, std::integral_constant<int, j < 8 ? j : 0>{});
                });
            }
            if constexpr (i == 1) { dma_w(a0, dk0, C0{}); dma_w(a0, dk0, C1{}); }
            if constexpr (i == 2) dma_w(a0, dk0, std::integral_constant<int, 2>{});
            if constexpr (i == 3) dma_w(a0, dk0, std::integral_constant<int, 3>{});
            if constexpr (END && i == 1) load_scales(m0, n0);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto rotate = [&]() {
        const int b0 = a0, b1 = a1;
        a0 = a2; a1 = a3; a2 = a4; a3 = b0; a4 = b1;
    };

    // copy position: two K-tiles ahead of the compute position; past the last tile the stream re-reads that tile
    int dkt = 2 % ktiles, dseq = 2 / ktiles;
    aim(0);
    static_for<0, 4>([&](auto jc) { dma_x(a0, 0, jc); });
    static_for<0, 4>([&](auto jc) { dma_w(a1, 0, jc); });
    static_for<0, 4>([&](auto jc) { dma_x(a2, BK, jc); });
    static_for<0, 4>([&](auto jc) { dma_w(a3, BK, jc); });
    if (dseq == 1 && my_tiles > 1) aim(1);
    __builtin_amdgcn_s_waitcnt(kWaitVm8);
    __syncthreads();
    static_for<0, 8>([&](auto ic) { read_one(a0, a1, C0{}, ic); });

    auto advance_copy = [&]() {
        if (++dkt == ktiles) {
            dkt = 0;
            if (++dseq < my_tiles) aim(dseq);
        }
    };

    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    for (int seq = 0; seq < my_tiles; ++seq) {
        int m0, n0;
        tile_at(seq, m0, n0);
        ktile(C1{}, C0{}, dkt * BK, m0, n0, seq == 0);
        rotate(); advance_copy();
        for (int kt = 1; kt + 1 < ktiles; ++kt) {
            ktile(C0{}, C0{}, dkt * BK, m0, n0, true);
            rotate(); advance_copy();
        }
        ktile(C0{}, C1{}, dkt * BK, m0, n0, true);
        rotate(); advance_copy();

        // ---- drain: a4 is free until this workgroup's own copies of the stream's next K-tile but one ----
        const int row = lane & 31;
        const int wswz = (row >> 1) & 7;
        const int rr = lane >> 3, rc = lane & 7;
        if constexpr (GATE) {
            // the two wavefronts of a row half share 64 rows x 128 bytes: each writes the 64 bytes per row of its 32
            // output columns, then (barrier) each streams out 32 whole rows
            uint8_t* stage = smem + a4 + wm * (64 * 128);
            uint8_t* wr = stage + row * 128 + khalf * 8;
#pragma unroll
            for (int b = 0; b < 2; ++b) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float c4[4] = {cs[0][g].x, cs[0][g].y, cs[0][g].z, cs[0][g].w};
                    const float u4[4] = {cs[1][g].x, cs[1][g].y, cs[1][g].z, cs[1][g].w};
                    float v[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        // the reference rounds gate and up to bf16 before the SiLU product
                        const uint32_t gu = pack_bf16x2_hw(acc[0][b][g * 4 + q] * (sa[b] * c4[q]), acc[1][b][g * 4 + q] * (sa[b] * u4[q]));
                        v[q] = fast_silu(bf16_lo(gu)) * bf16_hi(gu);
                    }
                    *reinterpret_cast<uint2*>(wr + b * 32 * 128 + (((wn * 4 + g) ^ wswz) << 4)) =
                        make_uint2(pack_bf16x2_hw(v[0], v[1]), pack_bf16x2_hw(v[2], v[3]));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            // every copy in flight is waited for before the first store (stores and copies share one counter); the tile
            // that follows skips the wait of its first K-tile
            __builtin_amdgcn_s_waitcnt(kWaitVm0);
            __syncthreads();
            const uint8_t* rdp0 = stage + (wn * 32 + rr) * 128 + ((rc ^ (rr >> 1)) << 4);
            const uint8_t* rdp1 = stage + (wn * 32 + rr) * 128 + ((rc ^ (rr >> 1) ^ 4) << 4);
            uint8_t* cu = reinterpret_cast<uint8_t*>(p.C + static_cast<size_t>(m0 + wm * 64 + wn * 32) * p.ldc + n0);
            const uint32_t coff = (static_cast<uint32_t>(rr) * static_cast<uint32_t>(p.ldc) + rc * 8u) * 2u;
            const size_t cstep = static_cast<size_t>(p.ldc) * 16;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 v = *reinterpret_cast<const uint4*>(((i & 1) ? rdp1 : rdp0) + i * 8 * 128);
                if (m0 + wm * 64 + wn * 32 + rr + i * 8 < p.M) {
                    const u32x4 vv = {v.x, v.y, v.z, v.w};
                    __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>(cu + i * cstep + coff));
                }
            }
        } else {
            // per 32 output rows: 32 rows x 128 bytes in this wavefront's own 4 KiB, then out as whole lines
            uint8_t* stage = smem + a4 + wave * (32 * BK);
            uint8_t* wr = stage + row * 128 + khalf * 8;
            const uint8_t* rdp0 = stage + rr * 128 + ((rc ^ (rr >> 1)) << 4);
            const uint8_t* rdp1 = stage + rr * 128 + ((rc ^ (rr >> 1) ^ 4) << 4);
            uint8_t* cu = reinterpret_cast<uint8_t*>(p.C + static_cast<size_t>(m0 + wm * 64) * p.ldc + n0 + wn * 64);
            const uint32_t coff = (static_cast<uint32_t>(rr) * static_cast<uint32_t>(p.ldc) + rc * 8u) * 2u;
            const size_t cstep = static_cast<size_t>(p.ldc) * 16;
#pragma unroll
            for (int b = 0; b < 2; ++b) {
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const float c4[4] = {cs[a][g].x, cs[a][g].y, cs[a][g].z, cs[a][g].w};
                        float v[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) v[q] = acc[a][b][g * 4 + q] * (sa[b] * c4[q]);
                        *reinterpret_cast<uint2*>(wr + (((a * 4 + g) ^ wswz) << 4)) =
                            make_uint2(pack_bf16x2_hw(v[0], v[1]), pack_bf16x2_hw(v[2], v[3]));
                    }
                __builtin_amdgcn_sched_barrier(0);
                if (b == 0) __builtin_amdgcn_s_waitcnt(kWaitVm0);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint4 v = *reinterpret_cast<const uint4*>(((i & 1) ? rdp1 : rdp0) + i * 8 * 128);
                    if (m0 + wm * 64 + b * 32 + rr + i * 8 < p.M) {
                        const u32x4 vv = {v.x, v.y, v.z, v.w};
                        __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>(cu + (b * 4 + i) * cstep + coff));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        static_for<0, 8>([&](auto ic) { read_one(a0, a1, C0{}, ic); });
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
}

// ---- block-scaled ring kernel ---------------------------------------------------------------
// The block-scaled GEMM on the persistent direct-to-LDS structure.  Needs K % 128 == 0, K >= 384,
// N % 256 == 0, operands smaller than 4 GiB, K / 128 <= 256.
// A K-tile is one scale group: its partial products start from a zero C operand and are folded into running
// sums as sum += part * (sa[m, kt] * sb[n / 128, kt]).  The fold is vector-ALU work in the inner loop (one
// multiply-add per accumulator element and K-tile), so this kernel runs TWO wavefronts per SIMD: the folds of
// one hide behind the MFMAs of the other, and with a 256-register budget per wavefront the MFMAs write their
// results to ordinary VGPRs, where the fold can read them (reading accumulation registers stalls while an MFMA
// is in flight).  Workgroup tile 128 x 256 x 128, eight wavefronts 2 x 4, each 64 x 64 = 2 x 2 MFMA tiles:
// sums 64 registers, partial products 64, two operand sets 64.
// LDS: three stages of (X 16 KiB + W 32 KiB); K-tile g lives in stage g % 3, K-tiles g+1 and g+2 are resident or
// landing, and the copies of K-tile g+3 go into stage g % 3 right after the barrier that ends its use.  The
// activation scales of a K-tile travel with it (one 4-byte copy per row into the stage's scale row), the
// weight-block scales of a tile (one per K-tile) are copied once per tile; the scale factors are therefore
// read from LDS and never wait on the copy pipeline.
constexpr int kBsThreads = 512;
constexpr int kBsX = BSM * BK;                          // 16 KiB
constexpr int kBsW = BN * BK;                           // 32 KiB
constexpr int kBsStage = kBsX + kBsW;                   // 48 KiB
constexpr int kBsSa = 3 * kBsStage;                     // activation scales: 3 stages x 128 floats
constexpr int kBsSb = kBsSa + 3 * BSM * 4;              // weight-block scales: 2 tile parities x 2 column blocks x 256 floats
constexpr int kBsMaxKb = 256;
constexpr int kBsLds = kBsSb + 2 * 2 * kBsMaxKb * 4;    // 153,088 bytes
// seven copy instructions per wavefront and K-tile (2 X, 4 W, 1 scales): waits leave one or two K-tiles in flight
constexpr int kWaitVm7 = 0x0f77, kWaitVm14 = 0x0f7e;

__global__ __launch_bounds__(kBsThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void k_gemm_nt_block_ring(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // 0..7
    const int wm = wave >> 2, wn = wave & 3;
    const int ktiles = p.K / BK;          // >= 3, checked by the launcher; also the number of scale groups along K
    const int total_tiles = p.tiles_m * p.tiles_n;
    int my_tiles, lin0, lstep;
    if (gridDim.x % kXcds == 0) {
        const int per = (total_tiles + kXcds - 1) / kXcds;
        const int x = blockIdx.x % kXcds, i = blockIdx.x / kXcds;
        lstep = gridDim.x / kXcds;
        const int cnt = max(0, min(per, total_tiles - x * per));
        my_tiles = (cnt - i + lstep - 1) / lstep;
        lin0 = x * per + i;
    } else {
        lstep = gridDim.x;
        my_tiles = (total_tiles - static_cast<int>(blockIdx.x) + lstep - 1) / lstep;
        lin0 = blockIdx.x;
    }
    if (my_tiles <= 0) return;
    auto tile_at = [&](int seq, int& m0, int& n0) {
        int tm, tn;
        tile_coords(lin0 + seq * lstep, p.tiles_m, p.tiles_n, tm, tn);
        m0 = tm * BSM;
        n0 = tn * BN;
    };

    // ---- global -> LDS: wave w copies X rows [16w, 16w+16), W rows [32w, 32w+32), the scales of X rows [16w, 16w+16) ----
    const int lrow = lane >> 3, lslot = lane & 7;
    uint32_t xoff[2], woff[4], saoff = 0;              // per-lane byte offsets
    const uint8_t* sbsrc = nullptr;                    // the tile's rows of weight-block scales
    auto aim = [&](int seq) {
        int m0, n0;
        tile_at(seq, m0, n0);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = wave * 16 + j * 8 + lrow;
            xoff[j] = static_cast<uint32_t>(min(m0 + row, p.M - 1)) * static_cast<uint32_t>(p.lda) + (lslot ^ swz(row)) * 16;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = wave * 32 + j * 8 + lrow;
            woff[j] = static_cast<uint32_t>(min(n0 + row, p.N - 1)) * static_cast<uint32_t>(p.ldb) + (lslot ^ swz(row)) * 16;
        }
        saoff = static_cast<uint32_t>(min(m0 + wave * 16 + (lane & 15), p.M - 1)) * static_cast<uint32_t>(ktiles) * 4u;
        sbsrc = reinterpret_cast<const uint8_t*>(p.sb + static_cast<size_t>((n0 >> 7) + (wave & 1)) * ktiles);
    };
    uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    auto dma16 = [&](uint32_t dst, uint32_t voff, const uint8_t* base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(dst), "v"(voff), "s"(base) : "memory");
    };
    // 4-byte copies by the low 16 lanes only: lane l lands at dst + 4 l.  The execution mask is narrowed and then set
    // back to all ones inside the statement; every call site is in wavefront-uniform control flow with all 64 lanes
    // active, so "all ones" is what it was.
    auto dma4_lo16 = [&](uint32_t dst, uint32_t voff, const uint8_t* base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_mov_b32 exec_lo, 0xffff\n\ts_mov_b32 exec_hi, 0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\t"
                     "s_mov_b32 exec_lo, -1\n\ts_mov_b32 exec_hi, -1\n\ts_nop 0"
                     :: "s"(dst), "v"(voff), "s"(base) : "memory");
    };
    auto dma4 = [&](uint32_t dst, uint32_t voff, const uint8_t* base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" :: "s"(dst), "v"(voff), "s"(base) : "memory");
    };
    // copy J (0..6) of the K-tile at K offset k0 (scale group kt) into the stage at `stage` (scale row sidx)
    auto copy_one = [&](int stage, int sidx, int k0, int kt, auto jc) {
        constexpr int J = decltype(jc)::value;
        if constexpr (J < 2)      dma16(lds0 + stage + (wave * 16 + J * 8) * BK, xoff[J], p.A + k0);
        else if constexpr (J < 6) dma16(lds0 + stage + kBsX + (wave * 32 + (J - 2) * 8) * BK, woff[J - 2], p.B + k0);
        else                      dma4_lo16(lds0 + kBsSa + sidx * (BSM * 4) + wave * 64, saoff, reinterpret_cast<const uint8_t*>(p.sa + kt));
    };
    // the weight-block scales of the tile the stream has just turned to: up to four copies of 64 floats by waves 0 and 1
    // (one per column block), into the half of the scale table selected by the tile's parity
    auto copy_sb = [&](int parity) {
        if (wave < 2) {
            for (int c = 0; c * 64 < ktiles; ++c) {
                const uint32_t v = static_cast<uint32_t>(min(c * 64 + lane, ktiles - 1)) * 4u;
                dma4(lds0 + kBsSb + (parity * 2 + wave) * (kBsMaxKb * 4) + c * 256, v, sbsrc);
            }
        }
    };

    // ---- LDS -> MFMA operands ----
    const int frow = lane & 31, khalf = lane >> 5, fs = swz(frow);
    int rd[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 2; ++j) rd[h][j] = frow * BK + (((h * 4 + khalf * 2 + j) ^ fs) << 4);
    const uint8_t* xrd = smem + wm * 64 * BK;
    const uint8_t* wrd = smem + kBsX + wn * 64 * BK;

    v16f part[2][2];      // [weight tile][activation tile]: this K-tile's partial products
    v16f sum[2][2];       // running sums, already scaled
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) sum[a][b][r] = 0.0f;
    v8i wq[2][2], xq[2][2];       // two operand sets: k-half h of any K-tile lives in set h
    auto put = [](v8i& dst, int half, const uint4 v) {
        dst[4 * half + 0] = (int)v.x; dst[4 * half + 1] = (int)v.y; dst[4 * half + 2] = (int)v.z; dst[4 * half + 3] = (int)v.w;
    };
    // read I (0..7) of k-half H from the stage at `stage`: w0 x0 x1 w1, two reads each
    auto read_one = [&](int stage, auto hc, auto ic) {
        constexpr int H = decltype(hc)::value, I = decltype(ic)::value;
        constexpr int t = I >> 1, half = I & 1;
        const int r = rd[H][half];
        if constexpr (t == 0)      put(wq[H][0], half, *reinterpret_cast<const uint4*>(wrd + stage + r));
        else if constexpr (t <= 2) put(xq[H][t - 1], half, *reinterpret_cast<const uint4*>(xrd + stage + (t - 1) * 32 * BK + r));
        else                       put(wq[H][1], half, *reinterpret_cast<const uint4*>(wrd + stage + 32 * BK + r));
    };
    auto mfma_one = [&](auto hc, auto ic) {
        constexpr int H = decltype(hc)::value, I = decltype(ic)::value;
        constexpr int a = I >> 1, b = I & 1;
        v16f c = part[a][b];
        if constexpr (H == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) c[r] = 0.0f;
        }
        part[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wq[H][a], xq[H][b], c, 0, 0, 0, 0, 0, 0);
    };
    // fold accumulator tile I of the K-tile whose factors are f[0], f[1] into the sums
    auto fold_one = [&](const float (&f)[2], auto ic) {
        constexpr int I = decltype(ic)::value;
        constexpr int a = I >> 1, b = I & 1;
        // volatile: the folds must stay between the MFMAs where they are written (the producing MFMA is at least
        // three MFMAs back there), not be gathered at the end of the loop body
        const float fv = f[b];
#pragma unroll
        for (int r = 0; r < 16; r += 8) {
            float v0 = sum[a][b][r], v1 = sum[a][b][r + 1], v2 = sum[a][b][r + 2], v3 = sum[a][b][r + 3];
            float v4 = sum[a][b][r + 4], v5 = sum[a][b][r + 5], v6 = sum[a][b][r + 6], v7 = sum[a][b][r + 7];
            const float p0 = part[a][b][r], p1 = part[a][b][r + 1], p2 = part[a][b][r + 2], p3 = part[a][b][r + 3];
            const float p4 = part[a][b][r + 4], p5 = part[a][b][r + 5], p6 = part[a][b][r + 6], p7 = part[a][b][r + 7];
            asm volatile("v_fmac_f32 %0, %8, %16\n\tv_fmac_f32 %1, %9, %16\n\tv_fmac_f32 %2, %10, %16\n\tv_fmac_f32 %3, %11, %16\n\t"
                         "v_fmac_f32 %4, %12, %16\n\tv_fmac_f32 %5, %13, %16\n\tv_fmac_f32 %6, %14, %16\n\tv_fmac_f32 %7, %15, %16"
                         : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                         : "v"(p0), "v"(p1), "v"(p2), "v"(p3), "v"(p4), "v"(p5), "v"(p6), "v"(p7), "v"(fv));
            sum[a][b][r] = v0; sum[a][b][r + 1] = v1; sum[a][b][r + 2] = v2; sum[a][b][r + 3] = v3;
            sum[a][b][r + 4] = v4; sum[a][b][r + 5] = v5; sum[a][b][r + 6] = v6; sum[a][b][r + 7] = v7;
        }
    };
    // the same fold in plain arithmetic, for the end of a tile, where the last MFMA has only just been issued
    auto fold_plain = [&](const float (&f)[2], auto ic) {
        constexpr int I = decltype(ic)::value;
        constexpr int a = I >> 1, b = I & 1;
#pragma unroll
        for (int r = 0; r < 16; ++r) sum[a][b][r] = __builtin_fmaf(part[a][b][r], f[b], sum[a][b][r]);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;

    int s0 = 0, s1 = kBsStage, s2 = 2 * kBsStage;      // stage offsets of K-tiles g, g+1, g+2
    int i0 = 0, i1 = 1, i2 = 2;                        // and their indices (for the scale rows)
    float f[2] = {0.0f, 0.0f};                         // factors of the K-tile whose partial products are still to be folded

    // One K-tile g at position kt of its tile.  FOLD: the previous K-tile's partial products are folded, each tile
    // right before the MFMA that overwrites it (not for a tile's first K-tile).  After the barrier the copies of
    // K-tile g+3 (K offset dk0, position dkt of its tile) start.
    // END: a tile's last K-tile: its copies are left to the caller (the epilogue stages the output in the stage they go to).
    auto ktile = [&](auto fold_c, auto end_c, int kt, int parity, int dk0, int dkt) {
        constexpr bool FOLD = decltype(fold_c)::value != 0, END = decltype(end_c)::value != 0;
        // step (g,0): 4 MFMAs from a zero C, the operand reads of (g,1)
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if constexpr (FOLD) fold_one(f, ic);
            mfma_one(C0{}, ic);
            read_one(s0, C1{}, std::integral_constant<int, 2 * i>{});
            read_one(s0, C1{}, std::integral_constant<int, 2 * i + 1>{});
            __builtin_amdgcn_sched_barrier(0);
        });
        // this K-tile's factors: read before the barrier, after which its scale row may be overwritten
        const float sbv = *reinterpret_cast<const float*>(smem + kBsSb + (parity * 2 + (wn >> 1)) * (kBsMaxKb * 4) + kt * 4);
#pragma unroll
        for (int b = 0; b < 2; ++b)
            f[b] = *reinterpret_cast<const float*>(smem + kBsSa + i0 * (BSM * 4) + (wm * 64 + b * 32 + (lane & 31)) * 4) * sbv;
        // step (g,1)
        mfma_one(C1{}, C0{});
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitVm7);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        static_for<1, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            mfma_one(C1{}, ic);
            // 8 reads and 7 copies over three slots
            static_for<0, 3>([&](auto jc) {
                constexpr int j = (i - 1) * 3 + decltype(jc)::value;
                if constexpr (j < 8) read_one(s1, C0{}, std::integral_constant<int, j < 8 ? j : 0>{});
                if constexpr (j < 7 && !END) copy_one(s0, i0, dk0, dkt, std::integral_constant<int, j < 7 ? j : 0>{});
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto rotate = [&]() {
        const int t = s0, u = i0;
        s0 = s1; s1 = s2; s2 = t;
        i0 = i1; i1 = i2; i2 = u;
    };

    // prologue: K-tiles 0, 1, 2 of the stream in flight, K-tile 0 landed and visible, operands (0,0) in set 0
    aim(0);
    copy_sb(0);
    static_for<0, 7>([&](auto jc) { copy_one(s0, i0, 0, 0, jc); });
    static_for<0, 7>([&](auto jc) { copy_one(s1, i1, BK, 1, jc); });
    static_for<0, 7>([&](auto jc) { copy_one(s2, i2, 2 * BK, 2, jc); });
    __builtin_amdgcn_s_waitcnt(kWaitVm14);
    __syncthreads();
    static_for<0, 8>([&](auto ic) { read_one(s0, C0{}, ic); });

    // copy position: three K-tiles ahead of the compute position (ktiles >= 3, so at most one tile ahead); past the
    // last tile the stream re-reads that tile and what it copies is never used
    int dkt = 3 % ktiles, dseq = 3 / ktiles;
    if (dseq == 1) {
        if (my_tiles > 1) aim(1);
        copy_sb(1);
    }
    auto advance_copy = [&]() {
        if (++dkt == ktiles) {
            dkt = 0;
            if (++dseq < my_tiles) aim(dseq);
            copy_sb(dseq & 1);
        }
    };

    const int khalf4 = khalf * 4;
    const bool vec_ok = (p.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 7u) == 0);
    const bool lines_ok = (p.ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 15u) == 0);        // whole 128-byte lines of C per row of a wavefront's tile
    for (int seq = 0; seq < my_tiles; ++seq) {
        int m0, n0;
        tile_at(seq, m0, n0);
        const int parity = seq & 1;
        ktile(C0{}, C0{}, 0, parity, dkt * BK, dkt);
        rotate(); advance_copy();
        for (int kt = 1; kt + 1 < ktiles; ++kt) {
            ktile(C1{}, C0{}, kt, parity, dkt * BK, dkt);
            rotate(); advance_copy();
        }
        ktile(C1{}, C1{}, ktiles - 1, parity, dkt * BK, dkt);
        // the last K-tile's partial products, then the sums leave as bf16
        static_for<0, 4>([&](auto ic) { fold_plain(f, ic); });
        if (lines_ok) {
            // A lane holds four consecutive columns of one row per quad: written from there a store instruction would
            // cover 32 rows with 16 bytes each.  The wavefront turns its 64 x 64 outputs round in LDS instead, 32 rows
            // at a time (128-byte rows, 16-byte chunks xor-swizzled by row), and stores whole lines, eight rows per
            // instruction.  The staging area is the 4 KiB of the stage just finished that this wavefront's own weight
            // copies of the K-tile three ahead go to: nobody reads that stage after the K-tile's barrier, and the
            // copies are issued below, in program order after the last staging read.
            uint8_t* stg = smem + s0 + kBsX + wave * (32 * BK);
            const int srow = lane & 31, rrow = lane >> 3, rchunk = lane & 7;
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int b = 0; b < 2; ++b) {
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const uint32_t o01 = pack_bf16x2_hw(sum[a][b][g * 4 + 0], sum[a][b][g * 4 + 1]);
                        const uint32_t o23 = pack_bf16x2_hw(sum[a][b][g * 4 + 2], sum[a][b][g * 4 + 3]);
                        *reinterpret_cast<uint2*>(stg + srow * 128 + (((a * 4 + g) ^ (srow & 7)) << 4) + khalf * 8) = make_uint2(o01, o23);
#pragma unroll
                        for (int q = 0; q < 4; ++q) sum[a][b][g * 4 + q] = 0.0f;
                    }
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int row = rrow + 8 * t;
                    const uint4 v = *reinterpret_cast<const uint4*>(stg + row * 128 + ((rchunk ^ (row & 7)) << 4));
                    const int m = m0 + wm * 64 + b * 32 + row;
                    if (m < p.M) {
                        const u32x4 vv = {v.x, v.y, v.z, v.w};
                        *reinterpret_cast<u32x4*>(p.C + static_cast<size_t>(m) * p.ldc + n0 + wn * 64 + rchunk * 8) = vv;
                    }
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int m = m0 + wm * 64 + b * 32 + (lane & 31);
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int n = n0 + wn * 64 + a * 32 + g * 8 + khalf4;
                        const uint32_t o01 = pack_bf16x2_hw(sum[a][b][g * 4 + 0], sum[a][b][g * 4 + 1]);
                        const uint32_t o23 = pack_bf16x2_hw(sum[a][b][g * 4 + 2], sum[a][b][g * 4 + 3]);
                        if (m < p.M) {
                            uint16_t* crow = p.C + static_cast<size_t>(m) * p.ldc + n;
                            if (vec_ok) {
                                *reinterpret_cast<uint2*>(crow) = make_uint2(o01, o23);
                            } else {
                                crow[0] = static_cast<uint16_t>(o01 & 0xffffu); crow[1] = static_cast<uint16_t>(o01 >> 16);
                                crow[2] = static_cast<uint16_t>(o23 & 0xffffu); crow[3] = static_cast<uint16_t>(o23 >> 16);
                            }
                        }
#pragma unroll
                        for (int q = 0; q < 4; ++q) sum[a][b][g * 4 + q] = 0.0f;
                    }
            }
        }
        // the copies the last K-tile left out
        static_for<0, 7>([&](auto jc) { copy_one(s0, i0, dkt * BK, dkt, jc); });
        rotate(); advance_copy();
    }
    // the copies started past the end of the stream must have landed before the LDS is given back
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
}

// ---- naive kernel: any shape, any alignment; also the on-device cross-check ----
// one lane per output element, fp32 accumulate in k order
__global__ __launch_bounds__(256) void k_gemm_nt_naive(const GemmArgs p, int fmt, int epi, int scale_mode) {
    const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<long long>(p.M) * p.N) return;
    const int m = static_cast<int>(idx / p.N), n = static_cast<int>(idx % p.N);
    const uint8_t* a = p.A + static_cast<size_t>(m) * p.lda;
    const uint8_t* b = p.B + static_cast<size_t>(n) * p.ldb;
    const uint8_t* b2 = epi == EPI_SILU_GATE ? p.B2 + static_cast<size_t>(n) * p.ldb : nullptr;
    if (scale_mode == SCALE_BLOCK) {
        // per 128-group partial sums, each promoted with its own factor
        const int kb = (p.K + 127) / 128;
        float total = 0.0f;
        for (int g = 0; g < kb; ++g) {
            float part = 0.0f;
            for (int k = g * 128; k < min(p.K, g * 128 + 128); ++k)
                part = __builtin_fmaf((fmt & 1) ? e5m2_to_f32(a[k]) : e4m3_to_f32(a[k]), e4m3_to_f32(b[k]), part);
            total = __builtin_fmaf(part, p.sa[static_cast<size_t>(m) * kb + g] * p.sb[static_cast<size_t>(n / 128) * kb + g], total);
        }
        p.C[static_cast<size_t>(m) * p.ldc + n] = f32_to_bf16(total);
        return;
    }
    float acc = 0.0f, acc2 = 0.0f;
    for (int k = 0; k < p.K; ++k) {
        const float av = (fmt & 1) ? e5m2_to_f32(a[k]) : e4m3_to_f32(a[k]);
        acc = __builtin_fmaf(av, (fmt & 2) ? e5m2_to_f32(b[k]) : e4m3_to_f32(b[k]), acc);
        if (b2) acc2 = __builtin_fmaf(av, e4m3_to_f32(b2[k]), acc2);
    }
    const float sa = scale_mode == SCALE_TENSOR ? p.sa[0] : p.sa[m];
    const float sb = scale_mode == SCALE_TENSOR ? p.sb[0] : p.sb[n];
    float v = acc * (sa * sb);
    if (epi == EPI_ACCUM_F32) { p.Cf[static_cast<size_t>(m) * p.ldc + n] += v; return; }
    if (epi == EPI_ACCUM_BF16) v += bf16_to_f32(p.C[static_cast<size_t>(m) * p.ldc + n]);
    if (epi == EPI_BIAS) v = bf16_to_f32(f32_to_bf16(v)) + bf16_to_f32(p.bias[n]);
    if (epi == EPI_SILU_GATE) {
        const float su = scale_mode == SCALE_TENSOR ? p.sb2[0] : p.sb2[n];
        const float gate = bf16_to_f32(f32_to_bf16(v));
        const float up = bf16_to_f32(f32_to_bf16(acc2 * (sa * su)));
        v = (gate * stable_sigmoid(gate)) * up;
    }
    p.C[static_cast<size_t>(m) * p.ldc + n] = f32_to_bf16(v);
}

inline int num_cus() {
    static int n = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) return 256;
        return v;
    }();
    return n;
}

template <int FMT, int EPI, int SCALE>
int launch_tiled(const GemmArgs& p, hipStream_t st) {
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt<FMT, EPI, SCALE>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    });
    if (attr_err != hipSuccess) return static_cast<int>(attr_err);
    // the ring kernel addresses operand rows by 32-bit byte offsets
    bool ring_ok = p.K % BK == 0 && p.K >= 2 * BK && static_cast<size_t>(p.a_rows) * p.lda < (1ull << 32) &&
                   static_cast<size_t>(p.N) * p.ldb < (1ull << 32);
    if constexpr (EPI == EPI_ACCUM_F32) {
        // its drain adds into full-width fp32 tiles with 16-byte accesses
        ring_ok = ring_ok && p.N % BN == 0 && p.ldc % 4 == 0 && aligned16(p.Cf);
    }
    if constexpr (EPI == EPI_ACCUM_BF16) {
        // the same with 8-byte accesses to bf16 tiles
        ring_ok = ring_ok && p.N % BN == 0 && p.ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(p.C) & 7u) == 0;
    }
    if constexpr (EPI == EPI_NONE || EPI == EPI_BIAS || EPI == EPI_SILU_GATE) {
        // its drain writes full-width tiles with 16-byte stores and reads the channel descales as float4
        // (N may cut the last column tile short at a multiple of 8; the fused gate/up form interleaves two weight
        // matrices per tile and keeps whole tiles)
        ring_ok = ring_ok && (EPI == EPI_SILU_GATE ? p.N % (BN / 2) == 0 : p.N % 8 == 0 && p.N >= 8) && p.ldc % 8 == 0 && aligned16(p.C);
        if (SCALE == SCALE_ROWCOL)
            ring_ok = ring_ok && aligned16(p.sb) && p.sb_expert_stride % 4 == 0 && (EPI != EPI_SILU_GATE || aligned16(p.sb2));
        if (EPI == EPI_BIAS) ring_ok = ring_ok && aligned16(p.bias);
    }
    if (ring_ok && !p.force_staged) {
        static std::once_flag once_ring;
        static hipError_t ring_err = hipSuccess;
        std::call_once(once_ring, [] {
            ring_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_ring<FMT, EPI, SCALE>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kRingLds);
        });
        if (ring_err != hipSuccess) return static_cast<int>(ring_err);
        // persistent: one workgroup per CU (the kernel uses a CU's whole LDS and register file);
        // a grid that is a multiple of 8 keeps "position % 8 = XCD" true for every tile a workgroup walks
        const int total = p.tiles_m * p.tiles_n;     // grouped: tiles_m is the host-side upper bound of row tiles
        int grid = total < num_cus() ? total : num_cus();
        if (grid >= kXcds) grid -= grid % kXcds;
        if constexpr (EPI == EPI_NONE || EPI == EPI_BIAS || EPI == EPI_SILU_GATE) {
            // the bf16 epilogues on an even number of K-tiles: the kernel on the 16 x 16 x 128 MFMA
            if (!p.mfma32 && (p.K / BK) % 2 == 0) {
                static std::once_flag once16;
                static hipError_t err16 = hipSuccess;
                std::call_once(once16, [] {
                    err16 = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_ring16<FMT, EPI, SCALE>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, kRingLds);
                });
                if (err16 != hipSuccess) return static_cast<int>(err16);
                k_gemm_nt_ring16<FMT, EPI, SCALE><<<grid, kThreads, kRingLds, st>>>(p);
                return launch_status();
            }
        }
        k_gemm_nt_ring<FMT, EPI, SCALE><<<grid, kThreads, kRingLds, st>>>(p);
        return launch_status();
    }
    k_gemm_nt<FMT, EPI, SCALE><<<p.tiles_m * p.tiles_n, kThreads, kLdsBytes, st>>>(p);
    return launch_status();
}

// the duo kernel: E4M3 operands, per-row x per-channel scales, plain or SiLU-gate epilogue, whole column tiles
template <int EPI>
int launch_duo(GemmArgs p, hipStream_t st) {
    static std::once_flag once;
    static hipError_t err = hipSuccess;
    std::call_once(once, [] {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_duo<EPI, true>), hipFuncAttributeMaxDynamicSharedMemorySize, kDuoLds);
        if (err == hipSuccess)
            err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_duo<EPI, false>), hipFuncAttributeMaxDynamicSharedMemorySize, kDuoLds);
    });
    if (err != hipSuccess) return static_cast<int>(err);
    constexpr int out_bn = EPI == EPI_SILU_GATE ? DM / 2 : DM;
    p.tiles_m = (p.M + DM - 1) / DM;
    p.tiles_n = p.N / out_bn;
    const int total = p.tiles_m * p.tiles_n;
    int grid = total < 2 * num_cus() ? total : 2 * num_cus();
    if (grid >= kXcds) grid -= grid % kXcds;
    if (p.duo == 2) k_gemm_nt_duo<EPI, false><<<grid, kThreads, kDuoLds, st>>>(p);
    else            k_gemm_nt_duo<EPI, true><<<grid, kThreads, kDuoLds, st>>>(p);
    return launch_status();
}
inline bool duo_ok(const GemmArgs& p, int fmt, int epi, int scale_mode) {
    const int out_bn = epi == EPI_SILU_GATE ? DM / 2 : DM;
    return fmt == 0 && scale_mode == SCALE_ROWCOL && (epi == EPI_NONE || epi == EPI_SILU_GATE) && !p.tile_map && p.K % BK == 0 &&
           p.K >= 2 * BK && p.N % out_bn == 0 && p.ldc % 8 == 0 && aligned16(p.C) && aligned16(p.sb) &&
           (epi != EPI_SILU_GATE || aligned16(p.sb2)) && static_cast<size_t>(p.M) * p.lda < (1ull << 32) &&
           static_cast<size_t>(p.N) * p.ldb < (1ull << 32);
}

template <int FMT, int EPI>
int dispatch_scale(const GemmArgs& p, int scale_mode, hipStream_t st) {
    return scale_mode == SCALE_TENSOR ? launch_tiled<FMT, EPI, SCALE_TENSOR>(p, st)
                                      : launch_tiled<FMT, EPI, SCALE_ROWCOL>(p, st);
}
// forward family: activations E4M3 or E5M2, weights E4M3
template <int FMT>
int dispatch_epi(const GemmArgs& p, int epi, int scale_mode, hipStream_t st) {
    switch (epi) {
        case EPI_NONE: return dispatch_scale<FMT, EPI_NONE>(p, scale_mode, st);
        case EPI_BIAS: return dispatch_scale<FMT, EPI_BIAS>(p, scale_mode, st);
        default:       return dispatch_scale<FMT, EPI_SILU_GATE>(p, scale_mode, st);
    }
}

// one wavefront: the row tiles of every expert in expert order (lane = expert, prefix sums of the row and tile
// counts); each row tile's entry describes its expert: number, row range, first row tile, row-tile count
// (offsets == nullptr: the experts' rows lie back to back, the first rows are the running sum of the counts).
// total_rows is the caller's bound on the rows the compact buffers hold (the reference's callers pass
// rows * top_k, src/trainer.cu:6863): an expert's range is cut at it, so that counts which sum to more than the
// bound cannot send a tile past the end of those buffers.
__device__ __forceinline__ void build_tile_map_wave(const int* __restrict__ counts, const int* __restrict__ offsets,
                                                    int num_experts, int max_row_tiles, int total_rows,
                                                    int* __restrict__ tile_map, int lane) {
    int carry = 0, carry_rows = 0, written = 0;
    for (int e0 = 0; e0 < num_experts; e0 += 64) {
        const int e = e0 + lane;
        const int cnt = e < num_experts ? max(counts[e], 0) : 0;
        int incl_rows = cnt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int r = __shfl_up(incl_rows, off, 64);
            if (lane >= off) incl_rows += r;
        }
        const int first = offsets ? (e < num_experts ? offsets[e] : 0) : carry_rows + incl_rows - cnt;
        const int kept = first >= 0 && first < total_rows ? min(cnt, total_rows - first) : 0;
        const int nt = (kept + BM - 1) / BM;
        int incl = nt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (lane >= off) incl += v;
        }
        const int base = carry + incl - nt;
        if (base + nt <= max_row_tiles) {        // always true when the experts' ranges do not overlap
            for (int i = 0; i < nt; ++i) {
                int* w = tile_map + 1 + kMapWords * (base + i);
                w[0] = e; w[1] = first; w[2] = first + kept; w[3] = base; w[4] = nt;
            }
            if (nt > 0) written = max(written, base + nt);
        }
        carry += __shfl(incl, 63, 64);
        carry_rows += __shfl(incl_rows, 63, 64);
    }
    // experts are written in order, so the ones that fit form a prefix: the table ends with the last of them
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) written = max(written, __shfl_xor(written, off, 64));
    if (lane == 0) tile_map[0] = written;
}
__global__ __launch_bounds__(64) void k_build_tile_map(const int* __restrict__ counts, const int* __restrict__ offsets,
                                                       int num_experts, int max_row_tiles, int total_rows,
                                                       int* __restrict__ tile_map) {
    build_tile_map_wave(counts, offsets, num_experts, max_row_tiles, total_rows, tile_map, threadIdx.x);
}

// Everything an expert bank derives from (counts, row lists) in one launch.  Workgroup e < num_experts: the offset
// of expert e (the sum of the counts before it; stored when the caller wants the array), its row list copied into the compact index at that offset and,
// when slot_index is given, the inverse entries slot_index[row, e] = position.  The last workgroup: the tile table.
// Entries at or beyond total_rows (the size of the compact buffers) are left out.
__global__ __launch_bounds__(256) void k_bank_setup(const int* __restrict__ counts, const int* __restrict__ row_indices, int rows,
                                                    int num_experts, int max_row_tiles, int total_rows, int* __restrict__ offsets,
                                                    int* __restrict__ compact, int* __restrict__ slot_index,
                                                    int* __restrict__ tile_map) {
    const int e = blockIdx.x, tid = threadIdx.x;
    if (e == num_experts) {
        if (tid < 64) build_tile_map_wave(counts, nullptr, num_experts, max_row_tiles, total_rows, tile_map, tid);
        return;
    }
    __shared__ int part[4];
    int sum = 0;
    for (int i = tid; i < e; i += 256) sum += max(counts[i], 0);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if ((tid & 63) == 0) part[tid >> 6] = sum;
    __syncthreads();
    const int base = part[0] + part[1] + part[2] + part[3];
    if (tid == 0 && offsets) offsets[e] = base;
    const int n = min(counts[e], total_rows - base);      // may be negative: nothing is copied then
    const int* list = row_indices + static_cast<size_t>(e) * rows;
    for (int s = tid; s < n; s += 256) {
        const int row = list[s];
        compact[base + s] = row;
        if (slot_index) slot_index[static_cast<size_t>(row) * num_experts + e] = base + s;
    }
}

int gemm_nt(GemmArgs p, int fmt, int epi, int scale_mode, int force_naive, cf_stream_t stream) {
    if (p.M < 0 || p.N < 0 || p.K < 0) return CF_ERR_INVALID_ARG;
    if (p.M == 0 || p.N == 0) return CF_OK;
    if (!p.A || !p.B || !(epi == EPI_ACCUM_F32 ? (void*)p.Cf : (void*)p.C) || !p.sa || !p.sb) return CF_ERR_INVALID_ARG;
    if (epi < EPI_NONE || epi > EPI_ACCUM_BF16 || scale_mode < SCALE_TENSOR || scale_mode > SCALE_BLOCK)
        return CF_ERR_INVALID_ARG;
    if (scale_mode == SCALE_BLOCK && (epi != EPI_NONE || fmt != 0)) return CF_ERR_UNSUPPORTED;
    if (epi == EPI_BIAS && !p.bias) return CF_ERR_INVALID_ARG;
    if (epi == EPI_SILU_GATE && (!p.B2 || !p.sb2)) return CF_ERR_INVALID_ARG;
    if (p.lda < p.K || p.ldb < p.K || p.ldc < p.N) return CF_ERR_INVALID_ARG;
    hipStream_t st = as_stream(stream);
    p.a_rows = p.M;
    const bool tiled_ok = p.K > 0 && p.K % 16 == 0 && p.lda % 16 == 0 && p.ldb % 16 == 0 && aligned16(p.A) &&
                          aligned16(p.B) && (epi != EPI_SILU_GATE || aligned16(p.B2));
    if (force_naive || !tiled_ok) {
        const long long total = static_cast<long long>(p.M) * p.N;
        k_gemm_nt_naive<<<static_cast<unsigned>((total + 255) / 256), 256, 0, st>>>(p, fmt, epi, scale_mode);
        return launch_status();
    }
    if (scale_mode == SCALE_BLOCK) {
        static std::once_flag once;
        static hipError_t attr_err = hipSuccess;
        std::call_once(once, [] {
            attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_block),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kBlkLds);
        });
        if (attr_err != hipSuccess) return static_cast<int>(attr_err);
        p.tiles_m = (p.M + BSM - 1) / BSM;
        p.tiles_n = (p.N + BN - 1) / BN;
        const int kb = p.K / BK;
        const bool ring_ok = p.K % BK == 0 && kb >= 3 && kb <= kBsMaxKb && p.N % BN == 0 && !p.force_staged &&
                             static_cast<size_t>(p.M) * p.lda < (1ull << 32) && static_cast<size_t>(p.N) * p.ldb < (1ull << 32) &&
                             static_cast<size_t>(p.M) * kb * 4 < (1ull << 32);
        if (ring_ok) {
            static std::once_flag once_ring;
            static hipError_t ring_err = hipSuccess;
            std::call_once(once_ring, [] {
                ring_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_block_ring),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kBsLds);
            });
            if (ring_err != hipSuccess) return static_cast<int>(ring_err);
            const int total = p.tiles_m * p.tiles_n;
            int grid = total < num_cus() ? total : num_cus();
            if (grid >= kXcds) grid -= grid % kXcds;
            k_gemm_nt_block_ring<<<grid, kBsThreads, kBsLds, st>>>(p);
            return launch_status();
        }
        k_gemm_nt_block<<<p.tiles_m * p.tiles_n, kThreads, kBlkLds, st>>>(p);
        return launch_status();
    }
    const int out_bn = epi == EPI_SILU_GATE ? BN / 2 : BN;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + out_bn - 1) / out_bn;
    if (epi == EPI_ACCUM_F32 || epi == EPI_ACCUM_BF16) {
        // weight-gradient family: per-tensor scales only, any operand format pair
        if (scale_mode != SCALE_TENSOR) return CF_ERR_UNSUPPORTED;
        const bool f32 = epi == EPI_ACCUM_F32;
        switch (fmt & 3) {
            case 0: return f32 ? launch_tiled<0, EPI_ACCUM_F32, SCALE_TENSOR>(p, st) : launch_tiled<0, EPI_ACCUM_BF16, SCALE_TENSOR>(p, st);
            case 1: return f32 ? launch_tiled<1, EPI_ACCUM_F32, SCALE_TENSOR>(p, st) : launch_tiled<1, EPI_ACCUM_BF16, SCALE_TENSOR>(p, st);
            case 2: return f32 ? launch_tiled<2, EPI_ACCUM_F32, SCALE_TENSOR>(p, st) : launch_tiled<2, EPI_ACCUM_BF16, SCALE_TENSOR>(p, st);
            default: return f32 ? launch_tiled<3, EPI_ACCUM_F32, SCALE_TENSOR>(p, st) : launch_tiled<3, EPI_ACCUM_BF16, SCALE_TENSOR>(p, st);
        }
    }
    if (fmt & 2) return CF_ERR_UNSUPPORTED;     // forward weights are always E4M3
    if (p.duo && duo_ok(p, fmt, epi, scale_mode))
        return epi == EPI_SILU_GATE ? launch_duo<EPI_SILU_GATE>(p, st) : launch_duo<EPI_NONE>(p, st);
    return (fmt & 1) ? dispatch_epi<1>(p, epi, scale_mode, st) : dispatch_epi<0>(p, epi, scale_mode, st);
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_fp8_gemm_nt_bf16(int M, int N, int K, const void* A, int lda, int a_is_e5m2, const float* a_descale,
                        const void* B, const float* b_descale, uint16_t* C, int ldc, cf_stream_t stream) {
    GemmArgs p{};
    p.M = M; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(A); p.lda = lda;
    p.B = static_cast<const uint8_t*>(B); p.ldb = K;
    p.sa = a_descale; p.sb = b_descale;
    p.C = C; p.ldc = ldc;
    return gemm_nt(p, a_is_e5m2 ? 1 : 0, EPI_NONE, SCALE_TENSOR, 0, stream);
}

int cf_fp8_gemm_nt_bf16_ex(int M, int N, int K, const void* A, int lda, int a_is_e5m2, const float* a_descale,
                           const void* B, int ldb, const float* b_descale, int scale_mode, int epilogue,
                           const uint16_t* bias, const void* B_up, const float* b_up_descale, uint16_t* C,
                           int ldc, int flags, cf_stream_t stream) {
    GemmArgs p{};
    p.M = M; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(A); p.lda = lda;
    p.B = static_cast<const uint8_t*>(B); p.ldb = ldb;
    p.B2 = static_cast<const uint8_t*>(B_up);
    p.sa = a_descale; p.sb = b_descale; p.sb2 = b_up_descale;
    p.bias = bias;
    p.C = C; p.ldc = ldc;
    if (epilogue > EPI_SILU_GATE) return CF_ERR_INVALID_ARG;
    p.force_staged = (flags & CF_GEMM_FLAG_STAGED) != 0;
    p.duo = (flags & CF_GEMM_FLAG_DUO) ? ((flags & CF_GEMM_FLAG_DUO_IN_STEP) ? 2 : 1) : 0;
    p.mfma32 = (flags & CF_GEMM_FLAG_MFMA32) != 0;
    return gemm_nt(p, a_is_e5m2 ? 1 : 0, epilogue, scale_mode, flags & CF_GEMM_FLAG_NAIVE, stream);
}

// dW[M,N] += X^T . dY with both operands pre-transposed to K-contiguous rows:
// "A" = X^T [M,K] E4M3, "B" = dY^T [N,K] E5M2.
int cf_fp8_gemm_tn_accum_f32(int M, int N, int K, const void* Xt_e4m3, const float* ds_x, const void* dYt_e5m2,
                             const float* ds_dy, float* dW, int ldc_dw, cf_stream_t stream) {
    GemmArgs p{};
    p.M = M; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(Xt_e4m3); p.lda = K;
    p.B = static_cast<const uint8_t*>(dYt_e5m2); p.ldb = K;
    p.sa = ds_x; p.sb = ds_dy;
    p.Cf = dW; p.ldc = ldc_dw;
    return gemm_nt(p, 2, EPI_ACCUM_F32, SCALE_TENSOR, 0, stream);
}

int cf_fp8_gemm_tn_accum_bf16(int M, int N, int K, const void* Xt_e4m3, const float* ds_x, const void* dYt_e5m2,
                              const float* ds_dy, uint16_t* dW, int ldc_dw, cf_stream_t stream) {
    GemmArgs p{};
    p.M = M; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(Xt_e4m3); p.lda = K;
    p.B = static_cast<const uint8_t*>(dYt_e5m2); p.ldb = K;
    p.sa = ds_x; p.sb = ds_dy;
    p.C = dW; p.ldc = ldc_dw;
    return gemm_nt(p, 2, EPI_ACCUM_BF16, SCALE_TENSOR, 0, stream);
}

int cf_fp8_grouped_gemm_workspace_bytes(int total_rows, int num_experts, size_t* bytes) {
    if (total_rows < 0 || num_experts < 0 || !bytes) return CF_ERR_INVALID_ARG;
    const size_t max_row_tiles = static_cast<size_t>(total_rows) / BM + static_cast<size_t>(num_experts);
    *bytes = (1 + kMapWords * max_row_tiles) * sizeof(int);
    return CF_OK;
}

int cf_fp8_grouped_gemm_nt_bf16_ex(int total_rows, int N, int K, int num_experts, const int* d_counts,
                                   const int* d_offsets, const void* A, int a_rows, int lda, const int* d_a_row_index,
                                   const float* a_descale, const void* B, const float* b_descale, int scale_mode,
                                   int epilogue, const void* B_up, const float* b_up_descale, uint16_t* C, int ldc,
                                   void* d_workspace, size_t workspace_bytes, cf_stream_t stream) {
    return cf::grouped_gemm_nt_bf16(total_rows, N, K, num_experts, d_counts, d_offsets, A, a_rows, lda, d_a_row_index, a_descale, B,
                                    b_descale, scale_mode, epilogue, B_up, b_up_descale, C, ldc, d_workspace, workspace_bytes,
                                    true, 0, stream);
}

// ---- the grouped GEMM for callers that cannot allocate ---------------------------------------------
// The tile table lives in a fixed array in the library's device image instead of a caller's workspace.  Each GPU
// holds its own copy of the array at its own address; host code must not pass the array's name to a kernel (in
// host code that name is a stand-in, not a device address), so the address is looked up once per device with
// hipGetSymbolAddress and every use below goes through that pointer.
constexpr size_t kStaticMapBytes = 64 * 1024;            // 3276 row tiles: e.g. 64 experts and 820,000 selected rows
static __device__ __align__(256) unsigned char scratch[kStaticMapBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// the address of `scratch` on the current device; looked up on the first call per device
int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return CF_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!ptr) return CF_ERR_UNSUPPORTED;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return CF_OK;
}
}  // namespace

// Also the set-up call: it looks up the array's address on the current device, so that a later call of the entry point
// (under graph capture, say) finds it ready and makes no runtime query of its own.
int cf_fp8_grouped_gemm_static_max_bytes(size_t* bytes) {
    if (!bytes) return CF_ERR_INVALID_ARG;
    *bytes = kStaticMapBytes;
    void* ptr = nullptr;
    return static_scratch(&ptr);
}

int cf_fp8_grouped_gemm_nt_bf16_static(int total_rows, int N, int K, int num_experts, const int* d_counts,
                                       const int* d_offsets, const void* A, int a_rows, int lda, const int* d_a_row_index,
                                       const float* a_descale, const void* B, const float* b_descale, int scale_mode,
                                       int epilogue, const void* B_up, const float* b_up_descale, uint16_t* C, int ldc,
                                       cf_stream_t stream) {
    size_t need = 0;
    const int rc = cf_fp8_grouped_gemm_workspace_bytes(total_rows, num_experts, &need);
    if (rc != CF_OK) return rc;
    if (need > kStaticMapBytes) return CF_ERR_UNSUPPORTED;       // the table of this many row tiles does not fit the fixed array
    void* ptr = nullptr;
    const int sc = static_scratch(&ptr);
    if (sc != CF_OK) return sc;
    // The table is rebuilt from the counts by every call (k_build_tile_map writes the entry count and every entry the
    // GEMM reads), so nothing of the previous call's contents is used and nothing needs clearing.
    return cf::grouped_gemm_nt_bf16(total_rows, N, K, num_experts, d_counts, d_offsets, A, a_rows, lda, d_a_row_index, a_descale, B,
                                    b_descale, scale_mode, epilogue, B_up, b_up_descale, C, ldc, ptr, kStaticMapBytes,
                                    true, 0, stream);
}

}  // extern "C"

void cf::build_tile_map(const int* d_counts, const int* d_offsets, int num_experts, int max_row_tiles, int total_rows,
                        int* tile_map, hipStream_t stream) {
    k_build_tile_map<<<1, 64, 0, stream>>>(d_counts, d_offsets, num_experts, max_row_tiles, total_rows, tile_map);
}

void cf::bank_setup(const int* d_counts, const int* d_row_indices, int rows, int num_experts, int total_rows, int* d_offsets,
                    int* d_compact_index, int* d_slot_index, int* tile_map, hipStream_t stream) {
    k_bank_setup<<<num_experts + 1, 256, 0, stream>>>(d_counts, d_row_indices, rows, num_experts, total_rows / BM + num_experts,
                                                      total_rows, d_offsets, d_compact_index, d_slot_index, tile_map);
}

// build_map = false: d_workspace already holds the tile table of these counts and offsets (an earlier call of
// the same routing on the same stream built it); a_is_e5m2: the activations are E5M2 (plain epilogue only)
int cf::grouped_gemm_nt_bf16(int total_rows, int N, int K, int num_experts, const int* d_counts, const int* d_offsets,
                             const void* A, int a_rows, int lda, const int* d_a_row_index, const float* a_descale,
                             const void* B, const float* b_descale, int scale_mode, int epilogue, const void* B_up,
                             const float* b_up_descale, uint16_t* C, int ldc, void* d_workspace, size_t workspace_bytes,
                             bool build_map, int a_is_e5m2, cf_stream_t stream) {
    if (total_rows < 0 || N < 0 || K < 0 || num_experts < 0 || a_rows < 0) return CF_ERR_INVALID_ARG;
    if (a_is_e5m2 && epilogue != EPI_NONE) return CF_ERR_UNSUPPORTED;
    if (total_rows == 0 || N == 0 || num_experts == 0) return CF_OK;
    if (!d_counts || !d_offsets || !A || !B || !C || !a_descale || !b_descale || !d_workspace) return CF_ERR_INVALID_ARG;
    if (epilogue != EPI_NONE && epilogue != EPI_SILU_GATE) return CF_ERR_INVALID_ARG;
    if (epilogue == EPI_SILU_GATE && (!B_up || !b_up_descale)) return CF_ERR_INVALID_ARG;
    if (scale_mode != SCALE_TENSOR && scale_mode != SCALE_ROWCOL) return CF_ERR_INVALID_ARG;
    // per-tensor descales would need one device scalar per expert for the weights: not built.  Rejected before
    // anything is launched, so a refused call leaves the workspace untouched.
    if (scale_mode == SCALE_TENSOR) return CF_ERR_UNSUPPORTED;
    size_t need = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_rows, num_experts, &need);
    if (workspace_bytes < need || (reinterpret_cast<uintptr_t>(d_workspace) & 3u)) return CF_ERR_INVALID_ARG;
    // the grouped form runs on the ring kernel only
    if (K % BK != 0 || K < 2 * BK || lda % 16 != 0 || !aligned16(A) || !aligned16(B) ||
        (epilogue == EPI_SILU_GATE && !aligned16(B_up)) || lda < K || ldc < N ||
        static_cast<size_t>(a_rows) * lda >= (1ull << 32) || static_cast<size_t>(N) * K >= (1ull << 32) ||
        (epilogue == EPI_SILU_GATE ? N % (BN / 2) != 0 : N % 8 != 0) || N < 8 || ldc % 8 != 0 || !aligned16(C) || !aligned16(b_descale) ||
        (epilogue == EPI_SILU_GATE && !aligned16(b_up_descale)))
        return CF_ERR_UNSUPPORTED;
    hipStream_t st = as_stream(stream);
    const int max_row_tiles = total_rows / BM + num_experts;
    int* tile_map = static_cast<int*>(d_workspace);
    if (build_map) k_build_tile_map<<<1, 64, 0, st>>>(d_counts, d_offsets, num_experts, max_row_tiles, total_rows, tile_map);
    GemmArgs p{};
    p.M = total_rows; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(A); p.lda = lda;
    p.B = static_cast<const uint8_t*>(B); p.ldb = K;
    p.B2 = static_cast<const uint8_t*>(B_up);
    p.sa = a_descale; p.sb = b_descale; p.sb2 = b_up_descale;
    p.C = C; p.ldc = ldc;
    p.tile_map = tile_map;
    p.a_row_index = d_a_row_index;
    p.a_rows = a_rows;
    p.b_expert_stride = static_cast<long long>(N) * K;
    p.sb_expert_stride = scale_mode == SCALE_ROWCOL ? N : 0;
    const int out_bn = epilogue == EPI_SILU_GATE ? BN / 2 : BN;
    p.tiles_m = max_row_tiles;
    p.tiles_n = (N + out_bn - 1) / out_bn;
    if (a_is_e5m2) return launch_tiled<1, EPI_NONE, SCALE_ROWCOL>(p, st);
    return epilogue == EPI_SILU_GATE ? launch_tiled<0, EPI_SILU_GATE, SCALE_ROWCOL>(p, st)
                                     : launch_tiled<0, EPI_NONE, SCALE_ROWCOL>(p, st);
}

namespace cf {
namespace {
// the ring kernel and nothing else: for the forms that exist only there
template <int FMT, int EPI, int SCALE, int MX>
int launch_ring_only(const GemmArgs& p, hipStream_t st) {
    static std::once_flag once;
    static hipError_t err = hipSuccess;
    std::call_once(once, [] {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_nt_ring<FMT, EPI, SCALE, MX>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kRingLds);
    });
    if (err != hipSuccess) return static_cast<int>(err);
    const int total = p.tiles_m * p.tiles_n;
    int grid = total < num_cus() ? total : num_cus();
    if (grid >= kXcds) grid -= grid % kXcds;
    k_gemm_nt_ring<FMT, EPI, SCALE, MX><<<grid, kThreads, kRingLds, st>>>(p);
    return launch_status();
}
}  // namespace

// C[r, :] = (A[index[r], :] . B[expert(r)]^T) * (a_descale[0] * b_descale[0]) in fp32, rows grouped by expert as in
// grouped_gemm_nt_bf16; d_tile_map is the table build_tile_map made for these counts.  N % 4 == 0.
int grouped_gemm_nt_store_f32(int total_rows, int N, int K, int num_experts, const void* A, int a_rows, int lda,
                              const int* d_a_row_index, const float* a_descale, const void* B, const float* b_descale,
                              float* C, int ldc, const int* d_tile_map, int a_is_e5m2, cf_stream_t stream) {
    if (total_rows <= 0 || N <= 0 || num_experts <= 0) return CF_OK;
    if (!A || !B || !C || !a_descale || !b_descale || !d_tile_map) return CF_ERR_INVALID_ARG;
    if (K % BK != 0 || K < 2 * BK || lda % 16 != 0 || lda < K || !aligned16(A) || !aligned16(B) || N % 4 != 0 || ldc % 4 != 0 ||
        ldc < N || !aligned16(C) || static_cast<size_t>(a_rows) * lda >= (1ull << 32) || static_cast<size_t>(N) * K >= (1ull << 32))
        return CF_ERR_UNSUPPORTED;
    GemmArgs p{};
    p.M = total_rows; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(A); p.lda = lda;
    p.B = static_cast<const uint8_t*>(B); p.ldb = K;
    p.sa = a_descale; p.sb = b_descale;
    p.Cf = C; p.ldc = ldc;
    p.tile_map = d_tile_map;
    p.a_row_index = d_a_row_index;
    p.a_rows = a_rows;
    p.b_expert_stride = static_cast<long long>(N) * K;
    p.tiles_m = total_rows / BM + num_experts;
    p.tiles_n = (N + BN - 1) / BN;
    hipStream_t st = as_stream(stream);
    return a_is_e5m2 ? launch_ring_only<1, EPI_STORE_F32, SCALE_TENSOR, 0>(p, st)
                     : launch_ring_only<0, EPI_STORE_F32, SCALE_TENSOR, 0>(p, st);
}

// C[r, :] = a_descale[r] * b_descale[0] * sum_t 2^(-4 t) A[r, t*Kb : (t+1)*Kb] . B[expert(r)]^T, bf16 or fp32: the activation
// rows are `terms` E4M3 terms side by side (lda >= terms * Kb), B is [num_experts, N, Kb] E4M3, b_descale one scalar
// for all experts.  Kb % 128 == 0; terms * Kb >= 256.
int grouped_gemm_nt_terms(int total_rows, int N, int Kb, int terms, int num_experts, const void* A, int lda,
                          const float* a_descale, const void* B, const float* b_descale, void* C, int ldc, bool c_is_f32,
                          const int* d_tile_map, cf_stream_t stream) {
    if (total_rows <= 0 || N <= 0 || num_experts <= 0) return CF_OK;
    if (!A || !B || !C || !a_descale || !b_descale || !d_tile_map || terms < 1 || terms > 8) return CF_ERR_INVALID_ARG;
    const long long K = static_cast<long long>(terms) * Kb;
    if (Kb % BK != 0 || Kb < BK || K < 2 * BK || lda % 16 != 0 || lda < K || !aligned16(A) || !aligned16(B) || N % 8 != 0 || N < 8 ||
        ldc % 8 != 0 || ldc < N || !aligned16(C) ||
        static_cast<size_t>(total_rows) * lda >= (1ull << 32) || static_cast<size_t>(N) * Kb >= (1ull << 32))
        return CF_ERR_UNSUPPORTED;
    GemmArgs p{};
    p.M = total_rows; p.N = N; p.K = static_cast<int>(K);
    p.A = static_cast<const uint8_t*>(A); p.lda = lda;
    p.B = static_cast<const uint8_t*>(B); p.ldb = Kb;
    p.sa = a_descale; p.sb = b_descale;
    if (c_is_f32) p.Cf = static_cast<float*>(C);
    else p.C = static_cast<uint16_t*>(C);
    p.ldc = ldc;
    p.tile_map = d_tile_map;
    p.a_rows = total_rows;
    p.b_expert_stride = static_cast<long long>(N) * Kb;
    p.sb_expert_stride = 0;
    p.b_k_period = Kb;
    p.tiles_m = total_rows / BM + num_experts;
    p.tiles_n = (N + BN - 1) / BN;
    return c_is_f32 ? launch_ring_only<0, EPI_STORE_F32, SCALE_ROW, 1>(p, as_stream(stream))
                    : launch_ring_only<0, EPI_NONE, SCALE_ROW, 1>(p, as_stream(stream));
}
}  // namespace cf

extern "C" {

// Cross-check form of the accumulate GEMMs: any format pair, optional naive kernel.
int cf_fp8_gemm_nt_accum_f32_ex(int M, int N, int K, const void* A, int lda, int a_is_e5m2, const float* a_descale,
                                const void* B, int ldb, int b_is_e5m2, const float* b_descale, float* C, int ldc,
                                int flags, cf_stream_t stream) {
    GemmArgs p{};
    p.M = M; p.N = N; p.K = K;
    p.A = static_cast<const uint8_t*>(A); p.lda = lda;
    p.B = static_cast<const uint8_t*>(B); p.ldb = ldb;
    p.sa = a_descale; p.sb = b_descale;
    p.Cf = C; p.ldc = ldc;
    p.force_staged = (flags & CF_GEMM_FLAG_STAGED) != 0;
    return gemm_nt(p, (a_is_e5m2 ? 1 : 0) | (b_is_e5m2 ? 2 : 0), EPI_ACCUM_F32, SCALE_TENSOR,
                   flags & CF_GEMM_FLAG_NAIVE, stream);
}

}  // extern "C"
