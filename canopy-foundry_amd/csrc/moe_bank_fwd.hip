// The GELU expert bank of moe_grouped_expert_forward_fp8 (/root/reference/kernels/moe.cu:950-1127) as a pipeline of
// whole-matrix launches: the reference's contract (per-tensor descales, fp32 projections, erf GELU kept beyond bf16 and
// not re-quantized to one fp8 value, w * y added into bf16 `mixed`) with both projections on the FP8 matrix cores.
//
//   fc_in   grouped FP8 GEMM over the gathered token rows, fp32 out (nothing is rounded before the GELU)
//   split   GELU in fp32, then each row as THREE E4M3 terms under one per-row scale s = 448 / amax(row):
//             q0 = e4m3(g s), q1 = e4m3(16 (g s - q0)), q2 = e4m3(16 (16 (g s - q0) - q1)),
//           so g s = q0 + q1 / 16 + q2 / 256 to 2^-13 of g s (an E4M3 rounding leaves at most 2^-4 of a normal value,
//           each residual is exact in fp32): 12 to 13 significand bits where bf16 has 8
//   fc_out  one grouped FP8 GEMM over K = 3 Ie: the three terms side by side against the same weights, the
//           matrix cores weighting term t by 2^(-4 t) through the E8M0 scale of v_mfma_scale_f32_32x32x64_f8f6f4,
//           so the three partial products meet in one fp32 accumulator; fp32 out
//   add     mixed[row] = bf16(mixed[row] + w * y) over the row's experts in ascending order, y in fp32, one bf16
//           rounding per expert as in the reference's compare-and-swap add
//
// Against the reference: the sum order over experts is fixed here where the reference's adds land in any order.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "cf_fp8.h"
#include "common.hpp"
#include "internal.hpp"

namespace cf {
namespace {

constexpr int kSplitThreads = 256;
constexpr int kTerms = 3;

// Phi(v) = (1 + erf(v / sqrt 2)) / 2 from the rational-exponential form of erfc (Abramowitz & Stegun 7.1.26,
// absolute error 1.5e-7 on erf: fp32 round-off level): for v < 0 the small tail is computed directly, not as
// 1 - (something near 1).
__device__ __forceinline__ float gelu_tail_form(float v) {
    const float z = fabsf(v) * 0.70710678f;
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, z, 1.0f));
    float poly = __builtin_fmaf(1.061405429f, t, -1.453152027f);
    poly = __builtin_fmaf(poly, t, 1.421413741f);
    poly = __builtin_fmaf(poly, t, -0.284496736f);
    poly = __builtin_fmaf(poly, t, 0.254829592f);
    const float half_erfc = 0.5f * poly * t * __builtin_amdgcn_exp2f(-1.44269504f * z * z);      // erfc(z) / 2
    const float cdf = v >= 0.0f ? 1.0f - half_erfc : half_erfc;
    return v * cdf;
}

__device__ __forceinline__ float4 decode4_e4m3(uint32_t q) {
    const f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q), false);
    const f32x2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q), true);
    return make_float4(lo[0], lo[1], hi[0], hi[1]);
}

// One wavefront per row of the fp32 projections [rows, K] (K % 4 == 0, K <= 256 MAXS): GELU, the row's scale, and
// the three terms written side by side into out[row, 0:3K]; descale[row] = amax / 448.
template <int MAXS>
__global__ __launch_bounds__(kSplitThreads) void k_gelu_split3(const float* __restrict__ pre, int rows, int K,
                                                               uint8_t* __restrict__ out, float* __restrict__ descale) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (kSplitThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const float* pr = pre + static_cast<size_t>(row) * K;
    f32x4 raw[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = (s * 64 + lane) * 4;
        raw[s] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (k < K) raw[s] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pr + k));
    }
    float4 g[MAXS];
    float m = 0.0f;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        g[s] = make_float4(gelu_tail_form(raw[s][0]), gelu_tail_form(raw[s][1]), gelu_tail_form(raw[s][2]), gelu_tail_form(raw[s][3]));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(g[s].x), fabsf(g[s].y)), fmaxf(fabsf(g[s].z), fabsf(g[s].w))));
    }
    m = wave_max(m);
    const float a = fmaxf(m, 1e-12f);
    const float sc = 448.0f / a;
    if (lane == 0) descale[row] = a / 448.0f;
    uint8_t* orow = out + static_cast<size_t>(row) * (kTerms * static_cast<size_t>(K));
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = (s * 64 + lane) * 4;
        if (k >= K) continue;
        float4 v = make_float4(g[s].x * sc, g[s].y * sc, g[s].z * sc, g[s].w * sc);
#pragma unroll
        for (int t = 0; t < kTerms; ++t) {
            const uint32_t q = cvt4_fp8<false>(v.x, v.y, v.z, v.w);
            *reinterpret_cast<uint32_t*>(orow + static_cast<size_t>(t) * K + k) = q;
            if (t + 1 < kTerms) {
                const float4 d = decode4_e4m3(q);
                // the clamp of the encode matters for term 0 only (g s may exceed 448 by a rounding); either way the
                // difference is what the later terms have to carry
                v = make_float4((v.x - d.x) * 16.0f, (v.y - d.y) * 16.0f, (v.z - d.z) * 16.0f, (v.w - d.w) * 16.0f);
            }
        }
    }
}

struct FwdWs { size_t off[CF_MOE_FWD_WS_COUNT]; size_t slot_bytes, total; };
FwdWs fwd_layout(int rows, int total_rows, int num_experts, int H, int Ie, bool bf16_form = false) {
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    FwdWs w{};
    size_t map_bytes = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_rows, num_experts, &map_bytes);
    const size_t T = static_cast<size_t>(total_rows);
    size_t off = 0;
    w.off[CF_MOE_FWD_WS_TILE_MAP] = off; off = up(off + map_bytes);
    w.off[CF_MOE_FWD_WS_OFFSETS] = off; off = up(off + sizeof(int) * static_cast<size_t>(num_experts));
    w.off[CF_MOE_FWD_WS_INDEX] = off; off = up(off + sizeof(int) * T);
    // the (row, expert) -> compact row table of the last step; beyond 64 MiB that step searches the row lists instead
    w.slot_bytes = sizeof(int) * static_cast<size_t>(rows) * num_experts;
    if (w.slot_bytes > (64u << 20)) w.slot_bytes = 0;
    w.off[CF_MOE_FWD_WS_SLOT] = off; off = up(off + w.slot_bytes);
    w.off[CF_MOE_FWD_WS_PRE] = off; off = up(off + sizeof(float) * T * Ie);
    if (bf16_form) {
        // the GELU output as bf16, no scales
        w.off[CF_MOE_FWD_WS_SPLIT] = off; off = up(off + 2 * T * Ie);
        w.off[CF_MOE_FWD_WS_SPLIT_DESCALE] = off;
        w.off[CF_MOE_FWD_WS_Y] = off; off = up(off + sizeof(float) * T * H);
        w.off[CF_MOE_FWD_WS_X] = off;
    } else {
        w.off[CF_MOE_FWD_WS_SPLIT] = off; off = up(off + kTerms * T * Ie);
        w.off[CF_MOE_FWD_WS_SPLIT_DESCALE] = off; off = up(off + sizeof(float) * T);
        w.off[CF_MOE_FWD_WS_Y] = off; off = up(off + sizeof(float) * T * H);
        w.off[CF_MOE_FWD_WS_X] = off;
    }
    w.total = off;
    return w;
}

// the shapes the pipeline takes; everything else stays with the one-kernel forms
bool staged_shape(int H, int Ie) { return H % 128 == 0 && H >= 256 && Ie % 128 == 0 && Ie >= 128 && Ie <= 4096; }
bool staged_shape_bf16(int H, int Ie) { return H % 8 == 0 && Ie % 64 == 0; }

// GELU of the fp32 projections rounded to bf16, as the reference kernel parks it before fc_out
// (sh_fcin[j] = __float2bfloat16(g), kernels/moe.cu:845).  K % 4 == 0.
__global__ __launch_bounds__(kSplitThreads) void k_gelu_round_bf16(const float* __restrict__ pre, size_t rows, int K,
                                                                   uint16_t* __restrict__ out) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int kv = K / 4;
    const size_t n = rows * kv;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kSplitThreads + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * kSplitThreads) {
        const size_t r = i / kv;
        const int c = static_cast<int>(i - r * kv) * 4;
        const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pre + r * K + c));
        const float g[4] = {gelu_tail_form(v[0]), gelu_tail_form(v[1]), gelu_tail_form(v[2]), gelu_tail_form(v[3])};
        store_stream8(out + r * static_cast<size_t>(K) + c, make_uint2(pack_bf16x2_hw(g[0], g[1]), pack_bf16x2_hw(g[2], g[3])));
    }
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_moe_grouped_expert_forward_fp8_workspace(int rows, int total_selected_rows, int num_experts, int H, int Ie,
                                                size_t* offsets, size_t* bytes) {
    if (rows < 0 || total_selected_rows < 0 || num_experts < 0 || H < 0 || Ie < 0 || !bytes) return CF_ERR_INVALID_ARG;
    if (!staged_shape(H, Ie)) {          // the one-kernel forms need no workspace
        *bytes = 0;
        if (offsets)
            for (int i = 0; i < CF_MOE_FWD_WS_COUNT; ++i) offsets[i] = 0;
        return CF_OK;
    }
    const FwdWs w = fwd_layout(rows, total_selected_rows, num_experts, H, Ie);
    *bytes = w.total;
    if (offsets)
        for (int i = 0; i < CF_MOE_FWD_WS_COUNT; ++i) offsets[i] = w.off[i];
    return CF_OK;
}

int cf_moe_grouped_expert_forward_fp8_ws(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                         const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                         const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                         const void* d_fc_out_w, const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                         int H, int Ie, int num_experts, int total_selected_rows, void* d_workspace,
                                         size_t workspace_bytes, cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0 || total_selected_rows < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0 || Ie == 0 || total_selected_rows == 0) return CF_OK;
    if (!d_hidden || !d_fcin_descale || !d_route_weights || !d_counts || !d_row_indices || !d_fc_in_w || !d_fc_in_descale ||
        !d_fc_out_w || !d_fc_out_descale || !d_mixed)
        return CF_ERR_INVALID_ARG;
    const bool staged = staged_shape(H, Ie) && aligned16(d_hidden) && aligned16(d_fc_in_w) && aligned16(d_fc_out_w) &&
                        aligned16(d_mixed) && static_cast<size_t>(rows) * H < (1ull << 32) &&
                        static_cast<size_t>(total_selected_rows) * kTerms * Ie < (1ull << 32) &&
                        static_cast<size_t>(H) * Ie < (1ull << 32);
    if (!staged)
        return expert_forward_fp8_one_kernel(d_hidden, d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts, d_row_indices, d_fc_in_w,
                                             d_fc_in_descale, d_fc_out_w, d_fc_out_descale, d_mixed, rows, H, Ie, num_experts, stream);
    const FwdWs w = fwd_layout(rows, total_selected_rows, num_experts, H, Ie);
    if (!d_workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(d_workspace) & 255u)) return CF_ERR_INVALID_ARG;
    auto* base = static_cast<uint8_t*>(d_workspace);
    int* tile_map = reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_TILE_MAP]);
    int* offsets = reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_OFFSETS]);
    int* index = reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_INDEX]);
    int* slot = w.slot_bytes ? reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_SLOT]) : nullptr;
    float* pre = reinterpret_cast<float*>(base + w.off[CF_MOE_FWD_WS_PRE]);
    uint8_t* split = base + w.off[CF_MOE_FWD_WS_SPLIT];
    float* split_descale = reinterpret_cast<float*>(base + w.off[CF_MOE_FWD_WS_SPLIT_DESCALE]);
    float* y = reinterpret_cast<float*>(base + w.off[CF_MOE_FWD_WS_Y]);
    hipStream_t st = as_stream(stream);

    // the reference takes the row lists without their offsets; the tile table and the compact index need them
    bank_setup(d_counts, d_row_indices, rows, num_experts, total_selected_rows, offsets, index, slot, tile_map, st);
    int rc = launch_status();
    if (rc) return rc;
    rc = grouped_gemm_nt_store_f32(total_selected_rows, Ie, H, num_experts, d_hidden, rows, H, index, d_fcin_descale, d_fc_in_w,
                                   d_fc_in_descale, pre, Ie, tile_map, fcin_is_e5m2 ? 1 : 0, stream);
    if (rc) return rc;
    {
        const unsigned grid = ceil_div(static_cast<size_t>(total_selected_rows), kSplitThreads / 64);
        if (Ie <= 512)       k_gelu_split3<2><<<grid, kSplitThreads, 0, st>>>(pre, total_selected_rows, Ie, split, split_descale);
        else if (Ie <= 1024) k_gelu_split3<4><<<grid, kSplitThreads, 0, st>>>(pre, total_selected_rows, Ie, split, split_descale);
        else if (Ie <= 1536) k_gelu_split3<6><<<grid, kSplitThreads, 0, st>>>(pre, total_selected_rows, Ie, split, split_descale);
        else if (Ie <= 2048) k_gelu_split3<8><<<grid, kSplitThreads, 0, st>>>(pre, total_selected_rows, Ie, split, split_descale);
        else                 k_gelu_split3<16><<<grid, kSplitThreads, 0, st>>>(pre, total_selected_rows, Ie, split, split_descale);
        rc = launch_status();
        if (rc) return rc;
    }
    rc = grouped_gemm_nt_terms(total_selected_rows, H, Ie, kTerms, num_experts, split, kTerms * Ie, split_descale, d_fc_out_w,
                               d_fc_out_descale, y, H, true, tile_map, stream);
    if (rc) return rc;
    return unpermute_f32(d_mixed, y, d_route_weights, slot, d_counts, offsets, d_row_indices, rows, num_experts, H,
                         total_selected_rows, st);
}

// moe_grouped_expert_forward_bf16 (kernels.hpp:400-407) with a workspace: the same pipeline on bf16 operands.
// fc_in is one grouped bf16 GEMM that gathers the token rows in its operand fetch, fp32 output; the GELU output is
// rounded to bf16 for fc_out, as in the reference kernel (kernels/moe.cu:845); y stays fp32 until the ordered add.
int cf_moe_grouped_expert_forward_bf16_workspace(int rows, int total_selected_rows, int num_experts, int H, int Ie,
                                                 size_t* offsets, size_t* bytes) {
    if (rows < 0 || total_selected_rows < 0 || num_experts < 0 || H < 0 || Ie < 0 || !bytes) return CF_ERR_INVALID_ARG;
    if (!staged_shape_bf16(H, Ie)) {
        *bytes = 0;
        if (offsets)
            for (int i = 0; i < CF_MOE_FWD_WS_COUNT; ++i) offsets[i] = 0;
        return CF_OK;
    }
    const FwdWs w = fwd_layout(rows, total_selected_rows, num_experts, H, Ie, true);
    *bytes = w.total;
    if (offsets)
        for (int i = 0; i < CF_MOE_FWD_WS_COUNT; ++i) offsets[i] = w.off[i];
    return CF_OK;
}

int cf_moe_grouped_expert_forward_bf16_ws(const uint16_t* d_hidden, const float* d_route_weights, const int* d_counts,
                                          const int* d_offsets, const int* d_row_indices, const uint16_t* d_fc_in_w,
                                          const uint16_t* d_fc_out_w, uint16_t* d_mixed, int rows, int H, int Ie,
                                          int num_experts, int total_selected_rows, void* d_workspace, size_t workspace_bytes,
                                          cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0 || total_selected_rows < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0 || Ie == 0 || total_selected_rows == 0) return CF_OK;
    if (!d_hidden || !d_route_weights || !d_counts || !d_row_indices || !d_fc_in_w || !d_fc_out_w || !d_mixed) return CF_ERR_INVALID_ARG;
    const bool staged = staged_shape_bf16(H, Ie) && aligned16(d_hidden) && aligned16(d_fc_in_w) && aligned16(d_fc_out_w) &&
                        aligned16(d_mixed) && static_cast<size_t>(rows) * H < (1ull << 30) &&
                        static_cast<size_t>(total_selected_rows) * Ie < (1ull << 30) && static_cast<size_t>(H) * Ie < (1ull << 30);
    if (!staged)
        return expert_forward_bf16_one_kernel(d_hidden, d_route_weights, d_counts, d_row_indices, d_fc_in_w, d_fc_out_w, d_mixed, rows,
                                              H, Ie, num_experts, stream);
    const FwdWs w = fwd_layout(rows, total_selected_rows, num_experts, H, Ie, true);
    if (!d_workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(d_workspace) & 255u)) return CF_ERR_INVALID_ARG;
    auto* base = static_cast<uint8_t*>(d_workspace);
    int* tile_map = reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_TILE_MAP]);
    int* offsets = reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_OFFSETS]);
    int* index = reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_INDEX]);
    int* slot = w.slot_bytes ? reinterpret_cast<int*>(base + w.off[CF_MOE_FWD_WS_SLOT]) : nullptr;
    float* pre = reinterpret_cast<float*>(base + w.off[CF_MOE_FWD_WS_PRE]);
    uint16_t* split = reinterpret_cast<uint16_t*>(base + w.off[CF_MOE_FWD_WS_SPLIT]);
    float* y = reinterpret_cast<float*>(base + w.off[CF_MOE_FWD_WS_Y]);
    hipStream_t st = as_stream(stream);

    bank_setup(d_counts, d_row_indices, rows, num_experts, total_selected_rows, offsets, index, slot, tile_map, st);
    int rc = launch_status();
    if (rc) return rc;
    // the token permute rides in fc_in's operand fetch
    rc = grouped_gemm_bf16_nt(total_selected_rows, Ie, H, 1, num_experts, d_hidden, rows, H, index, d_fc_in_w, pre, Ie, true, tile_map,
                              stream);
    if (rc) return rc;
    {
        const size_t n = static_cast<size_t>(total_selected_rows) * (Ie / 4);
        const unsigned want = ceil_div(n, kSplitThreads);
        k_gelu_round_bf16<<<want < 16384u ? want : 16384u, kSplitThreads, 0, st>>>(pre, static_cast<size_t>(total_selected_rows), Ie, split);
        rc = launch_status();
        if (rc) return rc;
    }
    rc = grouped_gemm_bf16_nt(total_selected_rows, H, Ie, 1, num_experts, split, total_selected_rows, Ie, nullptr, d_fc_out_w, y, H,
                              true, tile_map, stream);
    if (rc) return rc;
    return unpermute_f32(d_mixed, y, d_route_weights, slot, d_counts, offsets, d_row_indices, rows, num_experts, H,
                         total_selected_rows, st);
}

}  // extern "C"
