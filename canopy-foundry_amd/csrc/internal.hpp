// Host-side entry points that the library's source files call across file boundaries (no kernels, no device code).
#pragma once
#include "common.hpp"

namespace cf {

// Word layout (4-byte words) of the device block behind a delayed-scaling activation slot (cf_act_slot): the ActSlot
// scalars of src/trainer.cu:3248-3278 plus two scratch words of the one-launch steady-state step, zero between calls.
namespace slotw {
enum { AMAX = 0, SCALE, DESCALE, SCALE_SNAP, DESCALE_SNAP, CALIB_MIN, CALIB_MAX, CURSOR = 8, COUNT = 9, RUNNING = 10, ARRIVED = 11,
       HISTORY = 16 };
}

// The grouped GEMM behind cf_fp8_grouped_gemm_nt_bf16_ex, for callers inside the library that run several
// projections over one routing: build_map = false reuses the tile table an earlier call left in d_workspace;
// a_is_e5m2 takes E5M2 activations (plain epilogue only).
int grouped_gemm_nt_bf16(int total_rows, int N, int K, int num_experts, const int* d_counts, const int* d_offsets,
                         const void* A, int a_rows, int lda, const int* d_a_row_index, const float* a_descale,
                         const void* B, const float* b_descale, int scale_mode, int epilogue, const void* B_up,
                         const float* b_up_descale, uint16_t* C, int ldc, void* d_workspace, size_t workspace_bytes,
                         bool build_map, int a_is_e5m2, cf_stream_t stream);

// Two forms that exist on the ring kernel only and take a tile table already built (gemm.hip): fp32 store with
// per-tensor descales and a row gather; the term-split form (activation rows = several E4M3 terms side by side,
// term t weighted 2^(-4 t) inside the matrix cores).
int grouped_gemm_nt_store_f32(int total_rows, int N, int K, int num_experts, const void* A, int a_rows, int lda,
                              const int* d_a_row_index, const float* a_descale, const void* B, const float* b_descale,
                              float* C, int ldc, const int* d_tile_map, int a_is_e5m2, cf_stream_t stream);
int grouped_gemm_nt_terms(int total_rows, int N, int Kb, int terms, int num_experts, const void* A, int lda,
                          const float* a_descale, const void* B, const float* b_descale, void* C, int ldc, bool c_is_f32,
                          const int* d_tile_map, cf_stream_t stream);
// The forward-pass form of the grouped bf16 GEMM (gemm_bf16.hip): C[r, :] = sum_t A[r, t*Kb:(t+1)*Kb] . B[expert(r)]^T,
// B [num_experts, N, Kb], C bf16 or fp32, tile table already built; d_a_row_index (may be null) gathers A's rows.
int grouped_gemm_bf16_nt(int total_rows, int N, int Kb, int terms, int num_experts, const uint16_t* A, int a_rows, int lda,
                         const int* d_a_row_index, const uint16_t* B, void* C, int ldc, bool c_is_f32, const int* d_tile_map,
                         cf_stream_t stream);
// The tile table of a grouped GEMM (k_build_tile_map in gemm.hip): tile_map[0] = number of row tiles of 256 rows,
// then per row tile (expert, its first row, its end row, its first row tile, its row-tile count), experts back to back.
// An expert's row range is cut at total_rows, the number of rows the compact buffers hold.
void build_tile_map(const int* d_counts, const int* d_offsets, int num_experts, int max_row_tiles, int total_rows,
                    int* tile_map, hipStream_t stream);
// The ordered weighted add of fp32 expert outputs into bf16 rows (moe.hip): d_slot_index null = search the row lists;
// slot_limit = the rows d_y holds, pairs whose slot lies at or beyond it are skipped.
int unpermute_f32(uint16_t* d_mixed, const float* d_y, const float* d_route_weights, const int* d_slot_index,
                  const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows, int num_experts, int H,
                  int slot_limit, hipStream_t st);
// One launch for what an expert bank derives from (counts, row lists [num_experts, rows]): the offsets, the compact
// row index, the (row, expert) -> compact row table (d_offsets and d_slot_index may be null) and the tile table of a grouped GEMM
// over total_rows rows.
void bank_setup(const int* d_counts, const int* d_row_indices, int rows, int num_experts, int total_rows, int* d_offsets,
                int* d_compact_index, int* d_slot_index, int* tile_map, hipStream_t stream);

// The one-kernel forms of the GELU expert bank (moe.hip): what cf_moe_grouped_expert_forward_fp8 / _bf16 run when no
// workspace is at hand.  Arguments checked by the callers.
int expert_forward_fp8_one_kernel(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2, const float* d_route_weights,
                                  const int* d_counts, const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                  const void* d_fc_out_w, const float* d_fc_out_descale, uint16_t* d_mixed, int rows, int H, int Ie,
                                  int num_experts, cf_stream_t stream);
int expert_forward_bf16_one_kernel(const uint16_t* d_hidden, const float* d_route_weights, const int* d_counts,
                                   const int* d_row_indices, const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w, uint16_t* d_mixed,
                                   int rows, int H, int Ie, int num_experts, cf_stream_t stream);

}  // namespace cf
