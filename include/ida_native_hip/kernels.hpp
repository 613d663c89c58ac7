// C++ shim over cf_fp8.h that re-declares the FP8 hot-path entry points of the reference's kernel
// library with their original names, argument order and error behaviour, over HIP types:
//
//   reference (include/ida_native/kernels.hpp)         here
//   __nv_bfloat16*                                      ida_native::bf16*  (16-bit storage, same layout)
//   cudaStream_t                                        hipStream_t
//   void return, throws std::runtime_error /            same: a non-zero C-ABI code becomes
//   std::invalid_argument (cuda_check.hpp:10-18,        std::invalid_argument (CF_ERR_INVALID_ARG) or
//   kernels/activations.cu:61-72)                       std::runtime_error (anything else)
//
// A translation unit of the reference trainer that included "ida_native/kernels.hpp" for these functions
// can include this header instead and link libcf_fp8.so.  Header-only; nothing here launches a kernel itself.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "cf_fp8.h"

namespace ida_native {

struct bf16 { std::uint16_t bits; };
static_assert(sizeof(bf16) == 2, "bf16 is 16-bit storage");

namespace hip_detail {
inline void check(int rc, const char* fn) {
    if (rc == CF_OK) return;
    if (rc == CF_ERR_INVALID_ARG) throw std::invalid_argument(std::string(fn) + ": invalid argument");
    if (rc == CF_ERR_UNSUPPORTED) throw std::runtime_error(std::string(fn) + ": unsupported shape or alignment");
    throw std::runtime_error(std::string(fn) + ": HIP error " + std::to_string(rc));
}
inline const std::uint16_t* u(const bf16* p) { return reinterpret_cast<const std::uint16_t*>(p); }
inline std::uint16_t* u(bf16* p) { return reinterpret_cast<std::uint16_t*>(p); }
}  // namespace hip_detail

#define CF_FWD(call) ::ida_native::hip_detail::check((call), __func__)

// ---- kernels.hpp:983-1052 (kernels/fp8.cu) ---------------------------------------------------------
inline void fp8_amax_bf16(const bf16* d_x, std::size_t n, float* d_amax, hipStream_t s) {
    CF_FWD(cf_fp8_amax_bf16(hip_detail::u(d_x), n, d_amax, s));
}
inline void fp8_pack_bf16_e4m3_raw(const bf16* d_x, std::uint8_t* d_out, float* d_amax, float* d_scale, float* d_descale,
                                   int* d_bad_count, std::size_t n, hipStream_t s) {
    CF_FWD(cf_fp8_pack_bf16_e4m3_raw(hip_detail::u(d_x), d_out, d_amax, d_scale, d_descale, d_bad_count, n, s));
}
inline void fp8_pack_bf16_e4m3_raw_and_dequant(const bf16* d_x, std::uint8_t* d_out, bf16* d_dequant, float* d_amax,
                                               float* d_scale, float* d_descale, int* d_bad_count, std::size_t n,
                                               hipStream_t s) {
    CF_FWD(cf_fp8_pack_bf16_e4m3_raw_and_dequant(hip_detail::u(d_x), d_out, hip_detail::u(d_dequant), d_amax, d_scale,
                                                 d_descale, d_bad_count, n, s));
}
inline void fp8_unpack_e4m3_raw_bf16(const std::uint8_t* d_in, const float* d_descale, bf16* d_out, std::size_t n,
                                     hipStream_t s) {
    CF_FWD(cf_fp8_unpack_e4m3_raw_bf16(d_in, d_descale, hip_detail::u(d_out), n, s));
}
inline void fp8_scale_from_amax(const float* d_amax, float fp8_max, float* d_scale, float* d_descale, hipStream_t s) {
    CF_FWD(cf_fp8_scale_from_amax(d_amax, fp8_max, d_scale, d_descale, s));
}
inline void fp8_quantize_e4m3(const bf16* d_x, void* d_out, const float* d_scale, std::size_t n, hipStream_t s) {
    CF_FWD(cf_fp8_quantize_e4m3(hip_detail::u(d_x), d_out, d_scale, n, s));
}
inline void fp8_quantize_e5m2(const bf16* d_x, void* d_out, const float* d_scale, std::size_t n, hipStream_t s) {
    CF_FWD(cf_fp8_quantize_e5m2(hip_detail::u(d_x), d_out, d_scale, n, s));
}
inline void fp8_quantize_transpose_e4m3(const bf16* d_w, void* d_out, const float* d_scale, int K, int N, hipStream_t s) {
    CF_FWD(cf_fp8_quantize_transpose_e4m3(hip_detail::u(d_w), d_out, d_scale, K, N, s));
}
inline void fp8_quant_and_transpose_e4m3(const bf16* d_in, void* d_act8_out, void* d_snap_out, const float* d_scale,
                                         int K, int N, hipStream_t s) {
    CF_FWD(cf_fp8_quant_and_transpose_e4m3(hip_detail::u(d_in), d_act8_out, d_snap_out, d_scale, K, N, s));
}
inline void fp8_quantize_e4m3_record(const bf16* d_x, void* d_out, const float* d_scale, float* d_amax, std::size_t n,
                                     hipStream_t s) {
    CF_FWD(cf_fp8_quantize_e4m3_record(hip_detail::u(d_x), d_out, d_scale, d_amax, n, s));
}
inline void fp8_quantize_e5m2_record(const bf16* d_x, void* d_out, const float* d_scale, float* d_amax, std::size_t n,
                                     hipStream_t s) {
    CF_FWD(cf_fp8_quantize_e5m2_record(hip_detail::u(d_x), d_out, d_scale, d_amax, n, s));
}
inline void fp8_clip_probe(const float* d_amax, const float* d_scale, float fp8_max, float* d_stats, hipStream_t s) {
    CF_FWD(cf_fp8_clip_probe(d_amax, d_scale, fp8_max, d_stats, s));
}
inline void fp8_elem_clip_count(const bf16* d_x, const float* d_scale, float fp8_max, std::size_t n, float* d_out,
                                hipStream_t s) {
    CF_FWD(cf_fp8_elem_clip_count(hip_detail::u(d_x), d_scale, fp8_max, n, d_out, s));
}
inline void fp8_update_delayed_scale(const float* d_amax, float fp8_max, float* d_scale, float* d_descale, float* d_history,
                                     int history_len, int* d_history_cursor, int* d_history_count, hipStream_t s) {
    CF_FWD(cf_fp8_update_delayed_scale(d_amax, fp8_max, d_scale, d_descale, d_history, history_len, d_history_cursor,
                                       d_history_count, s));
}

// ---- kernels.hpp:159-165, 243-247 (kernels/activations.cu, kernels/moe.cu) -------------------------------
inline void swiglu_forward(const bf16* d_gate, const bf16* d_up, bf16* d_out, int N, hipStream_t stream) {
    CF_FWD(cf_swiglu_forward(hip_detail::u(d_gate), hip_detail::u(d_up), hip_detail::u(d_out), N, stream));
}
inline void swiglu_backward(const bf16* d_grad_out, const bf16* d_gate, const bf16* d_up, bf16* d_grad_gate,
                            bf16* d_grad_up, int N, hipStream_t stream) {
    CF_FWD(cf_swiglu_backward(hip_detail::u(d_grad_out), hip_detail::u(d_gate), hip_detail::u(d_up),
                              hip_detail::u(d_grad_gate), hip_detail::u(d_grad_up), N, stream));
}
inline void col_sum_strided_bf16(const bf16* d_in, float* d_out_accum, int rows, int cols, int row_stride, int base,
                                 hipStream_t stream) {
    CF_FWD(cf_col_sum_strided_bf16(hip_detail::u(d_in), d_out_accum, rows, cols, row_stride, base, stream));
}
inline void bias_add_strided_bf16(bf16* d_inout, const bf16* d_bias, int rows, int cols, int row_stride, int base,
                                  hipStream_t stream) {
    CF_FWD(cf_bias_add_strided_bf16(hip_detail::u(d_inout), hip_detail::u(d_bias), rows, cols, row_stride, base, stream));
}

// ---- kernels.hpp:117-120 (kernels/rmsnorm.cu) ---------------------------------------------------------------
inline void rmsnorm_forward(const bf16* d_x, const bf16* d_scale, bf16* d_out, float* d_rms, int rows, int H, float eps,
                            hipStream_t stream) {
    CF_FWD(cf_rmsnorm_forward(hip_detail::u(d_x), hip_detail::u(d_scale), hip_detail::u(d_out), d_rms, rows, H, eps, stream));
}

// ---- kernels.hpp:571-585 (kernels/cross_entropy.cu) -------------------------------------------------------
inline void cross_entropy_count_valid(const int32_t* d_labels, int n, int* d_n_valid, hipStream_t stream) {
    CF_FWD(cf_cross_entropy_count_valid(d_labels, n, d_n_valid, stream));
}
inline void cross_entropy_fwd_bwd_chunk(const bf16* d_logits, const int32_t* d_labels, float* d_loss_out, bf16* d_grad,
                                        int rows, int V, const int* d_n_valid, hipStream_t stream) {
    CF_FWD(cf_cross_entropy_fwd_bwd_chunk(hip_detail::u(d_logits), d_labels, d_loss_out, hip_detail::u(d_grad), rows, V, d_n_valid, stream));
}

// ---- kernels.hpp:193, 313-317, 340-343, 361-423 (kernels/cross_entropy.cu, kernels/moe.cu) -----------------
inline void softmax_inplace_f32(float* d_x, int rows, int cols, hipStream_t stream) {
    CF_FWD(cf_softmax_inplace_f32(d_x, rows, cols, stream));
}
inline void moe_topk_route_f32(float* d_scores, int rows, int num_experts, int top_k, hipStream_t stream,
                               float* d_row_sum_save = nullptr, float* d_scores_save = nullptr,
                               bool normalize_topk = true) {
    CF_FWD(cf_moe_topk_route_f32(d_scores, rows, num_experts, top_k, stream, d_row_sum_save, d_scores_save,
                                 normalize_topk ? 1 : 0));
}
inline void moe_scale_accumulate_bf16(bf16* d_mixed, const bf16* d_term, const float* d_route_weights, int rows,
                                      int expert_idx, int num_experts, int H, hipStream_t stream) {
    CF_FWD(cf_moe_scale_accumulate_bf16(hip_detail::u(d_mixed), hip_detail::u(d_term), d_route_weights, rows, expert_idx,
                                        num_experts, H, stream));
}
inline void moe_build_expert_row_lists(const float* d_route_weights, int* d_counts, int* d_row_indices, int rows,
                                       int num_experts, hipStream_t stream) {
    CF_FWD(cf_moe_build_expert_row_lists(d_route_weights, d_counts, d_row_indices, rows, num_experts, stream));
}
inline void moe_gather_rows_bf16(const bf16* d_src, bf16* d_dst, const int* d_row_indices, int n_rows, int width,
                                 hipStream_t stream) {
    CF_FWD(cf_moe_gather_rows_bf16(hip_detail::u(d_src), hip_detail::u(d_dst), d_row_indices, n_rows, width, stream));
}
inline void moe_gather_rows_u8(const std::uint8_t* d_src, std::uint8_t* d_dst, const int* d_row_indices, int n_rows,
                               int width, hipStream_t stream) {
    CF_FWD(cf_moe_gather_rows_u8(d_src, d_dst, d_row_indices, n_rows, width, stream));
}
inline void moe_scatter_accumulate_rows_bf16(bf16* d_mixed, const bf16* d_compact, const float* d_route_weights,
                                             const int* d_row_indices, int n_rows, int expert_idx, int num_experts, int H,
                                             hipStream_t stream) {
    CF_FWD(cf_moe_scatter_accumulate_rows_bf16(hip_detail::u(d_mixed), hip_detail::u(d_compact), d_route_weights,
                                               d_row_indices, n_rows, expert_idx, num_experts, H, stream));
}
// ---- kernels.hpp:334, kernels/moe.cu:623-674,740-767,1148-1167: the selected-expert backward's kernels ------
inline void gelu_forward(const bf16* d_x, bf16* d_out, std::size_t n, hipStream_t stream) {
    CF_FWD(cf_gelu_forward_bf16(hip_detail::u(d_x), hip_detail::u(d_out), n, stream));
}
inline void gelu_backward(const bf16* d_pre, const bf16* d_grad_post, bf16* d_grad_pre, std::size_t n, hipStream_t stream) {
    CF_FWD(cf_gelu_backward_bf16(hip_detail::u(d_pre), hip_detail::u(d_grad_post), hip_detail::u(d_grad_pre), n, stream));
}
inline void moe_row_dot_selected_bf16(const bf16* d_a_full, const bf16* d_b_compact, float* d_out, const int* d_row_indices,
                                      int n_rows, int H, int out_stride, int out_col, hipStream_t stream) {
    CF_FWD(cf_moe_row_dot_selected_bf16(hip_detail::u(d_a_full), hip_detail::u(d_b_compact), d_out, d_row_indices, n_rows, H,
                                        out_stride, out_col, stream));
}
inline void moe_gather_scale_rows_bf16(const bf16* d_src, bf16* d_dst, const float* d_route_weights, const int* d_row_indices,
                                       int n_rows, int expert_idx, int num_experts, int H, hipStream_t stream) {
    CF_FWD(cf_moe_gather_scale_rows_bf16(hip_detail::u(d_src), hip_detail::u(d_dst), d_route_weights, d_row_indices, n_rows,
                                         expert_idx, num_experts, H, stream));
}
inline void moe_scatter_add_rows_bf16(bf16* d_dst_full, const bf16* d_src_compact, const int* d_row_indices, int n_rows, int H,
                                      hipStream_t stream) {
    CF_FWD(cf_moe_scatter_add_rows_bf16(hip_detail::u(d_dst_full), hip_detail::u(d_src_compact), d_row_indices, n_rows, H, stream));
}
inline void moe_expert_offsets_from_counts(const int* d_counts, int* d_offsets, int num_experts, hipStream_t stream) {
    CF_FWD(cf_moe_expert_offsets_from_counts(d_counts, d_offsets, num_experts, stream));
}
inline void moe_grouped_expert_forward_bf16(const bf16* d_hidden, const float* d_route_weights, const int* d_counts,
                                            const int* d_offsets, const int* d_row_indices, const bf16* d_fc_in_w,
                                            const bf16* d_fc_out_w, bf16* d_mixed, int rows, int H, int Ie, int num_experts,
                                            int total_selected_rows, hipStream_t stream) {
    CF_FWD(cf_moe_grouped_expert_forward_bf16(hip_detail::u(d_hidden), d_route_weights, d_counts, d_offsets, d_row_indices,
                                              hip_detail::u(d_fc_in_w), hip_detail::u(d_fc_out_w), hip_detail::u(d_mixed), rows, H,
                                              Ie, num_experts, total_selected_rows, stream));
}
inline void moe_grouped_expert_forward_fp8(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                           const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                           const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                           const void* d_fc_out_w, const float* d_fc_out_descale, bf16* d_mixed, int rows,
                                           int H, int Ie, int num_experts, int total_selected_rows, hipStream_t stream) {
    CF_FWD(cf_moe_grouped_expert_forward_fp8(d_hidden, d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts, d_offsets,
                                             d_row_indices, d_fc_in_w, d_fc_in_descale, d_fc_out_w, d_fc_out_descale,
                                             hip_detail::u(d_mixed), rows, H, Ie, num_experts, total_selected_rows, stream));
}
// The bf16 bank with a workspace slice: both projections as whole-matrix grouped bf16 GEMMs where the shape allows.
inline size_t moe_grouped_expert_forward_bf16_workspace_bytes(int rows, int H, int Ie, int num_experts, int total_selected_rows) {
    size_t bytes = 0;
    CF_FWD(cf_moe_grouped_expert_forward_bf16_workspace(rows, total_selected_rows, num_experts, H, Ie, nullptr, &bytes));
    return bytes;
}
inline void moe_grouped_expert_forward_bf16(const bf16* d_hidden, const float* d_route_weights, const int* d_counts,
                                            const int* d_offsets, const int* d_row_indices, const bf16* d_fc_in_w,
                                            const bf16* d_fc_out_w, bf16* d_mixed, int rows, int H, int Ie, int num_experts,
                                            int total_selected_rows, void* d_workspace, size_t workspace_bytes,
                                            hipStream_t stream) {
    CF_FWD(cf_moe_grouped_expert_forward_bf16_ws(hip_detail::u(d_hidden), d_route_weights, d_counts, d_offsets, d_row_indices,
                                                 hip_detail::u(d_fc_in_w), hip_detail::u(d_fc_out_w), hip_detail::u(d_mixed), rows,
                                                 H, Ie, num_experts, total_selected_rows, d_workspace, workspace_bytes, stream));
}
// The same call with a workspace slice (the trainer's arena can supply one): both projections then run as whole-matrix
// FP8 GEMMs where the shape allows.  moe_grouped_expert_forward_fp8_workspace_bytes gives the size (0: not needed).
inline size_t moe_grouped_expert_forward_fp8_workspace_bytes(int rows, int H, int Ie, int num_experts, int total_selected_rows) {
    size_t bytes = 0;
    CF_FWD(cf_moe_grouped_expert_forward_fp8_workspace(rows, total_selected_rows, num_experts, H, Ie, nullptr, &bytes));
    return bytes;
}
inline void moe_grouped_expert_forward_fp8(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                           const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                           const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                           const void* d_fc_out_w, const float* d_fc_out_descale, bf16* d_mixed, int rows,
                                           int H, int Ie, int num_experts, int total_selected_rows, void* d_workspace,
                                           size_t workspace_bytes, hipStream_t stream) {
    CF_FWD(cf_moe_grouped_expert_forward_fp8_ws(d_hidden, d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts, d_offsets,
                                                d_row_indices, d_fc_in_w, d_fc_in_descale, d_fc_out_w, d_fc_out_descale,
                                                hip_detail::u(d_mixed), rows, H, Ie, num_experts, total_selected_rows,
                                                d_workspace, workspace_bytes, stream));
}

// ---- the static GEMM / transpose helpers of src/trainer.cu, minus their Fp8Ctx argument ----------------------
// transpose_u8, src/trainer.cu:1441-1448
inline void transpose_u8(const void* in, void* out, int rows, int cols, hipStream_t s) {
    CF_FWD(cf_transpose_u8(in, out, rows, cols, s));
}
// lt_gemm_fp8_nt, src/trainer.cu:4498-4534; a_is_e5m2 replaces the cudaDataType_t a_type argument
inline void lt_gemm_fp8_nt(int M, int N, int K, const void* A, int lda, bool a_is_e5m2, const float* a_descale,
                           const void* B, const float* b_descale, bf16* C, int ldc, hipStream_t s) {
    CF_FWD(cf_fp8_gemm_nt_bf16(M, N, K, A, lda, a_is_e5m2 ? 1 : 0, a_descale, B, b_descale, hip_detail::u(C), ldc, s));
}
// lt_gemm_fp8_tn_accum_f32, src/trainer.cu:4596-4627 and :4670-4691
inline void lt_gemm_fp8_tn_accum_f32(int M, int N, int K, const void* Xt_e4m3, const float* ds_x, const void* dYt_e5m2,
                                     const float* ds_dy, float* dW, int ldc_dw, hipStream_t s) {
    CF_FWD(cf_fp8_gemm_tn_accum_f32(M, N, K, Xt_e4m3, ds_x, dYt_e5m2, ds_dy, dW, ldc_dw, s));
}
inline void lt_gemm_fp8_tn_accum_f32(int M, int N, int K, const void* Xt_e4m3, const float* ds_x, const void* dYt_e5m2,
                                     const float* ds_dy, bf16* dW, int ldc_dw, hipStream_t s) {
    CF_FWD(cf_fp8_gemm_tn_accum_bf16(M, N, K, Xt_e4m3, ds_x, dYt_e5m2, ds_dy, hip_detail::u(dW), ldc_dw, s));
}

// gemm_bf16 and gemm_bf16_tn_f32, src/trainer.cu:3069-3090 and :3116-3160, as the selected-expert backward calls
// them (:7727-7740): the cuBLAS handle becomes the stream, alpha is 1, beta is 0 for the input gradients and 1 for the
// weight gradients; any other pair throws.
inline void gemm_bf16(hipStream_t s, int M, int N, int K, float alpha, const bf16* A, int lda, const bf16* B, int ldb,
                      float beta, bf16* C, int ldc) {
    if (alpha != 1.0f || beta != 0.0f) throw std::invalid_argument("gemm_bf16: only alpha = 1, beta = 0 is built");
    CF_FWD(cf_gemm_bf16_nn(M, N, K, hip_detail::u(A), lda, hip_detail::u(B), ldb, hip_detail::u(C), ldc, s));
}
inline void gemm_bf16_tn_f32(hipStream_t s, int M, int N, int K, float alpha, const bf16* A, int lda, const bf16* B,
                             int ldb, float beta, float* C, int ldc) {
    if (alpha != 1.0f || beta != 1.0f) throw std::invalid_argument("gemm_bf16_tn_f32: only alpha = 1, beta = 1 is built");
    CF_FWD(cf_gemm_bf16_tn_accum_f32(M, N, K, hip_detail::u(A), lda, hip_detail::u(B), ldb, C, ldc, s));
}
inline void gemm_bf16_tn_f32(hipStream_t s, int M, int N, int K, float alpha, const bf16* A, int lda, const bf16* B,
                             int ldb, float beta, bf16* C, int ldc) {
    if (alpha != 1.0f || beta != 1.0f) throw std::invalid_argument("gemm_bf16_tn_f32: only alpha = 1, beta = 1 is built");
    CF_FWD(cf_gemm_bf16_tn_accum_bf16(M, N, K, hip_detail::u(A), lda, hip_detail::u(B), ldb, hip_detail::u(C), ldc, s));
}

#undef CF_FWD

}  // namespace ida_native
