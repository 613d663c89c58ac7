/*
 * cf_fp8.h -- C ABI of the MI355X (gfx950) FP8 hot-path library.
 *
 * Every entry point replaces one function of the reference's kernel library
 * (C++ free functions in namespace ida_native, declared in
 * include/ida_native/kernels.hpp of the reference tree) or one of the static
 * cuBLASLt wrappers in src/trainer.cu; the citation after each declaration
 * names it.  Conventions, all taken from the reference call sites:
 *   - every pointer is device memory owned by the caller, scalars included
 *     (amax / scale / descale / history / cursor / count are device scalars);
 *   - work is enqueued on `stream` (a hipStream_t passed as void*) and nothing
 *     synchronises;
 *   - bf16 tensors are passed as uint16_t*, fp8 tensors as void* / uint8_t*;
 *   - the library allocates no device memory; the only allocation is the
 *     small host object behind cf_act_slot_create (freed by
 *     cf_act_slot_destroy).  It keeps no state between calls and every entry
 *     point may be called from several host threads and streams at once on
 *     buffers that do not overlap, with one exception that says so where it is
 *     declared: cf_fp8_grouped_gemm_nt_bf16_static, whose tile table is a
 *     fixed array in the library's device image shared by all its calls on a
 *     GPU.  One-time kernel attribute set-up runs under std::call_once;
 *   - total_selected_rows / total_rows of the expert-bank entry points is an
 *     UPPER BOUND on the sum of the device-side counts, as the reference's
 *     callers pass it (rows * top_k, src/trainer.cu:6863): it sizes the
 *     compact buffers and the workspace; the true total is taken from the
 *     counts on the device.  Should the counts sum to more than the bound,
 *     the rows beyond it are left out (nothing is written or read past the
 *     buffers the bound sized) and the result misses their terms.
 * The reference functions return void and throw; the C ABI returns 0 on
 * success, a positive hipError_t when the runtime reports one, or a negative
 * CF_ERR_* code for an argument the kernels cannot honour.
 */
#ifndef CF_FP8_H
#define CF_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* cf_stream_t; /* hipStream_t */

#define CF_OK                 0
#define CF_ERR_INVALID_ARG   (-1)  /* null pointer with n > 0, negative size       */
#define CF_ERR_UNSUPPORTED   (-2)  /* shape / alignment outside what a kernel takes */

#define CF_E4M3_MAX 448.0f
#define CF_E5M2_MAX 57344.0f

/* library identification: returns a static string naming arch and build */
const char* cf_version(void);

/* ---- per-tensor quantize family: kernels/fp8.cu --------------------------- */

/* fp8_amax_bf16, kernels.hpp:983, kernels/fp8.cu:250-253.  Zeroes *d_amax then
 * max-reduces |x| into it. */
int cf_fp8_amax_bf16(const uint16_t* d_x, size_t n, float* d_amax, cf_stream_t stream);

/* fp8_scale_from_amax, kernels.hpp:1002, kernels/fp8.cu:255-259. */
int cf_fp8_scale_from_amax(const float* d_amax, float fp8_max, float* d_scale,
                           float* d_descale, cf_stream_t stream);

/* fp8_quantize_e4m3 / fp8_quantize_e5m2, kernels.hpp:1004-1007,
 * kernels/fp8.cu:261-279.  out[i] = cvt_rne_satfinite(f32(x[i]) * *d_scale). */
int cf_fp8_quantize_e4m3(const uint16_t* d_x, void* d_out, const float* d_scale,
                         size_t n, cf_stream_t stream);
int cf_fp8_quantize_e5m2(const uint16_t* d_x, void* d_out, const float* d_scale,
                         size_t n, cf_stream_t stream);

/* fp8_quantize_e4m3_record / _e5m2_record, kernels.hpp:1021-1026,
 * kernels/fp8.cu:310-330.  Quantizes with *d_scale and max-combines the amax
 * of the unscaled input into *d_amax (caller zeroes it). */
int cf_fp8_quantize_e4m3_record(const uint16_t* d_x, void* d_out, const float* d_scale,
                                float* d_amax, size_t n, cf_stream_t stream);
int cf_fp8_quantize_e5m2_record(const uint16_t* d_x, void* d_out, const float* d_scale,
                                float* d_amax, size_t n, cf_stream_t stream);

/* fp8_update_delayed_scale, kernels.hpp:1042-1052, kernels/fp8.cu:396-417. */
int cf_fp8_update_delayed_scale(const float* d_amax, float fp8_max, float* d_scale,
                                float* d_descale, float* d_history, int history_len,
                                int* d_history_cursor, int* d_history_count,
                                cf_stream_t stream);

/* The steady-state branch of fp8_quant_act (src/trainer.cu:4811-4851) in ONE launch instead of the reference's
 * two device-to-device copies, one memset and two kernels: quantize with *d_scale (the scale the previous call
 * left) while recording this tensor's amax; then, inside the same kernel, the pair the quantize used goes to
 * *d_scale_snapshot / *d_descale_snapshot (what the following GEMM dequantizes with), the amax to *d_amax, and
 * the history, cursor, count, *d_scale and *d_descale advance as fp8_update_delayed_scale does
 * (kernels/fp8.cu:105-142).  d_running_amax and d_arrived are two words of caller-owned device memory that
 * must be zero before the first call; every call leaves them zero again.  Calls on one state must not overlap. */
int cf_fp8_quantize_delayed_step(const uint16_t* d_x, void* d_out, size_t n, int is_e5m2,
                                 float* d_amax, float* d_scale, float* d_descale,
                                 float* d_scale_snapshot, float* d_descale_snapshot,
                                 float* d_history, int history_len, int* d_history_cursor,
                                 int* d_history_count, float* d_running_amax,
                                 unsigned int* d_arrived, cf_stream_t stream);

/* fp8_quantize_transpose_e4m3, kernels.hpp:1009-1010, kernels/fp8.cu:281-290.
 * w[K,N] bf16 -> out[N,K] E4M3. */
int cf_fp8_quantize_transpose_e4m3(const uint16_t* d_w, void* d_out, const float* d_scale,
                                   int K, int N, cf_stream_t stream);

/* fp8_quant_and_transpose_e4m3, kernels.hpp:1015-1017, kernels/fp8.cu:292-308.
 * in[K,N] bf16 -> act8[K,N] and snap[N,K], one read. */
int cf_fp8_quant_and_transpose_e4m3(const uint16_t* d_in, void* d_act8_out, void* d_snap_out,
                                    const float* d_scale, int K, int N, cf_stream_t stream);

/* transpose_u8, static at src/trainer.cu:1441-1448.  in[rows,cols] -> out[cols,rows]. */
int cf_transpose_u8(const void* d_in, void* d_out, int rows, int cols, cf_stream_t stream);

/* fp8_clip_probe / fp8_elem_clip_count, kernels.hpp:1033-1041,
 * kernels/fp8.cu:358-394. */
int cf_fp8_clip_probe(const float* d_amax, const float* d_scale, float fp8_max,
                      float* d_stats, cf_stream_t stream);
int cf_fp8_elem_clip_count(const uint16_t* d_x, const float* d_scale, float fp8_max,
                           size_t n, float* d_out, cf_stream_t stream);

/* fp8_pack_bf16_e4m3_raw / _raw_and_dequant / fp8_unpack_e4m3_raw_bf16,
 * kernels.hpp:988-1001, kernels/fp8.cu:491-528.  Byte contract of
 * include/ida_native/fp8_e4m3.hpp (nonfinite -> sign|0x7f and counted).
 * *d_bad_count is nonzero iff an input or a packed product was nonfinite. */
int cf_fp8_pack_bf16_e4m3_raw(const uint16_t* d_x, uint8_t* d_out, float* d_amax,
                              float* d_scale, float* d_descale, int* d_bad_count,
                              size_t n, cf_stream_t stream);
int cf_fp8_pack_bf16_e4m3_raw_and_dequant(const uint16_t* d_x, uint8_t* d_out,
                                          uint16_t* d_dequant, float* d_amax, float* d_scale,
                                          float* d_descale, int* d_bad_count, size_t n,
                                          cf_stream_t stream);
int cf_fp8_unpack_e4m3_raw_bf16(const uint8_t* d_in, const float* d_descale, uint16_t* d_out,
                                size_t n, cf_stream_t stream);

/* k_calib_minmax_update, static at src/trainer.cu:3789-3795. */
int cf_fp8_calib_minmax_update(const float* d_amax, float* d_cmin, float* d_cmax,
                               cf_stream_t stream);

/* ---- scale groups finer than per-tensor ------------------------------------
 * The reference scales per tensor only (kernels/fp8.cu:13-16); these apply the
 * same formula (kernels/fp8.cu:37-39,49) per row, per 1x128 group and per
 * 128x128 block, and to fp32 input, for the benchmark configurations that ask
 * for them.  Scale tensors are fp32: [rows], [rows, ceil(K/128)],
 * [ceil(rows/128), ceil(K/128)]. */
int cf_fp8_amax_f32(const float* d_x, size_t n, float* d_amax, cf_stream_t stream);
int cf_fp8_quantize_f32_e4m3(const float* d_x, void* d_out, const float* d_scale, size_t n,
                             cf_stream_t stream);
int cf_fp8_quantize_f32_e5m2(const float* d_x, void* d_out, const float* d_scale, size_t n,
                             cf_stream_t stream);
int cf_fp8_quantize_rows(const uint16_t* d_x, int rows, int K, int is_e5m2, void* d_out,
                         float* d_scale, float* d_descale, cf_stream_t stream);
int cf_fp8_quantize_block_1x128(const uint16_t* d_x, int rows, int K, void* d_out,
                                float* d_scale, float* d_descale, cf_stream_t stream);
int cf_fp8_quantize_block_128x128(const uint16_t* d_x, int rows, int K, void* d_out,
                                  float* d_scale, float* d_descale, cf_stream_t stream);

/* ---- elementwise epilogue ops (also fused into the GEMM epilogue) ---------- */

/* swiglu_forward, kernels.hpp:159-165, kernels/activations.cu:76-87.
 * n < 0 or a null pointer with n > 0 is CF_ERR_INVALID_ARG (the reference
 * throws std::invalid_argument, kernels/activations.cu:61-72). */
int cf_swiglu_forward(const uint16_t* d_gate, const uint16_t* d_up, uint16_t* d_out, int n,
                      cf_stream_t stream);
/* swiglu_backward, kernels.hpp:167-175, kernels/activations.cu:42-58, 89-106:
 * grad_gate = bf16((grad_out * up) * silu'(gate)), grad_up = bf16(grad_out * silu(gate)).
 * n < 0 or a null pointer with n > 0 is CF_ERR_INVALID_ARG, as the reference throws. */
int cf_swiglu_backward(const uint16_t* d_grad_out, const uint16_t* d_gate, const uint16_t* d_up,
                       uint16_t* d_grad_gate, uint16_t* d_grad_up, int n, cf_stream_t stream);
/* bias_add_strided_bf16, kernels.hpp:243-247, kernels/moe.cu:349-356. */
int cf_bias_add_strided_bf16(uint16_t* d_inout, const uint16_t* d_bias, int rows, int cols,
                             int row_stride, int base, cf_stream_t stream);
/* col_sum_strided_bf16, kernels.hpp:255-259, kernels/moe.cu:335-348, 357-364: the bias gradient,
 * out_accum[c] += sum over rows of in[row, base + c], the sum taken in fp32 in ascending row order
 * from zero (the reference's order, so the bits are the reference's). */
int cf_col_sum_strided_bf16(const uint16_t* d_in, float* d_out_accum, int rows, int cols,
                            int row_stride, int base, cf_stream_t stream);

/* ---- producers of the quantizer's input, fused with it ---------------------
 * The reference normalises, clips and quantizes an activation in four launches
 * (src/trainer.cu:6281-6304: rmsnorm_forward, act_row_clip, fp8_quant_act); the
 * fused forms below give the same bytes in one pass over the row.  All of them
 * follow the reference's reduction trees, so the bf16 results are bit-identical
 * to the launch sequence.  Shapes: H <= 16384 and min(H, 512) a multiple of 32
 * (the reference's full-mask shuffles are defined for whole 32-lane groups
 * only); anything else is CF_ERR_UNSUPPORTED.  Rows move as 16-byte vectors
 * when H % 8 == 0 and the row pointers are 16-byte aligned (fp8 rows 8-byte). */

/* rmsnorm_forward, kernels.hpp:117, kernels/rmsnorm.cu:13-54,101-108.
 * d_rms may be null.  d_out may alias d_x. */
int cf_rmsnorm_forward(const uint16_t* d_x, const uint16_t* d_scale, uint16_t* d_out, float* d_rms,
                       int rows, int H, float eps, cf_stream_t stream);
/* act_row_clip in its fixed-ceiling mode, src/trainer.cu:3968-3991 (static;
 * kernels :3822-3842, :3940-3958) without the optional statistics: rows whose
 * L2 norm exceeds `ceiling` are scaled down to it in place; ceiling <= 0 is a
 * no-op (:3974).  d_normsq[rows] receives the row sums of squares as the
 * reference's scratch does; may be null. */
int cf_act_row_clip_abs(uint16_t* d_x, int rows, int cols, float ceiling, float* d_normsq,
                        cf_stream_t stream);
/* rmsnorm_forward -> act_row_clip(ceiling) -> per-row quantize (cf_fp8_quantize_rows)
 * in one launch (the sequence at src/trainer.cu:6281-6304 with per-token scales).  d_normed (the bf16 normalised, clipped row, which the
 * reference keeps for the router and the weight gradient) and d_rms may be null. */
int cf_rmsnorm_clip_quantize_rows(const uint16_t* d_x, const uint16_t* d_scale, int rows, int H,
                                  float eps, float ceiling, int is_e5m2, uint16_t* d_normed,
                                  float* d_rms, void* d_q, float* d_row_scale,
                                  float* d_row_descale, cf_stream_t stream);
/* rmsnorm_forward -> act_row_clip(ceiling) -> fp8_quantize_e4m3_record /
 * _e5m2_record (kernels/fp8.cu:67-103, 310-330): quantize with *d_qscale and
 * raise *d_amax to the tensor's maximum (the caller zeroes it, as for
 * cf_fp8_quantize_e4m3_record). */
int cf_rmsnorm_clip_quantize_record(const uint16_t* d_x, const uint16_t* d_scale, int rows, int H,
                                    float eps, float ceiling, int is_e5m2, uint16_t* d_normed,
                                    float* d_rms, void* d_q, const float* d_qscale,
                                    float* d_amax, cf_stream_t stream);

/* ---- loss head: chunked cross-entropy, fused with the quantize of its gradient ---------
 * The FP8 head (src/trainer.cu:8015-8060) projects a chunk of rows onto the vocabulary with the NT GEMM above,
 * runs cross-entropy forward + backward in place, and quantizes the bf16 gradient to E5M2 for the input-gradient
 * GEMM.  exp / log run on the hardware units here, so gradients agree with a correctly rounded evaluation to one
 * bf16 ulp (CUDA's expf / logf bits are not reproducible either). */

/* cross_entropy_count_valid, kernels.hpp:571-573, kernels/cross_entropy.cu:201-219,281-287:
 * adds the number of labels >= 0 to *d_n_valid (the caller zeroes it). */
int cf_cross_entropy_count_valid(const int32_t* d_labels, int n, int* d_n_valid, cf_stream_t stream);
/* cross_entropy_fwd_bwd_chunk, kernels.hpp:577-585, kernels/cross_entropy.cu:225-305:
 * grad[r,v] = bf16((softmax(logits[r])[v] - (v == label[r])) / max(*n_valid, 1)), rows with a negative label get
 * zeros; *d_loss_out += -log(p_label + 1e-9) / max(*n_valid, 1) per valid row.  d_grad may alias d_logits. */
int cf_cross_entropy_fwd_bwd_chunk(const uint16_t* d_logits, const int32_t* d_labels, float* d_loss_out,
                                   uint16_t* d_grad, int rows, int V, const int* d_n_valid,
                                   cf_stream_t stream);
/* The same plus what fp8_quant_act does to the gradient in its steady state (src/trainer.cu:8053,
 * kernels/fp8.cu:86-103): d_grad8 = E5M2(bf16 gradient * *d_qscale), *d_amax raised to the gradient's
 * maximum (the caller zeroes it).  One pass over the logits instead of four. */
int cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(const uint16_t* d_logits, const int32_t* d_labels,
                                              float* d_loss_out, uint16_t* d_grad, void* d_grad8,
                                              const float* d_qscale, float* d_amax, int rows, int V,
                                              const int* d_n_valid, cf_stream_t stream);

/* ---- scaled FP8 GEMM -------------------------------------------------------
 * Replaces the reference's cuBLASLt wrappers, which are static functions of
 * src/trainer.cu bound to its Fp8Ctx (handle, workspace, plan cache); the
 * entry points take the same operands without the context.  fp32 accumulate. */

#define CF_SCALE_PER_TENSOR 0  /* a_descale[1], b_descale[1] (device scalars)   */
#define CF_SCALE_ROW_COL    1  /* a_descale[M] per token, b_descale[N] per channel */
#define CF_SCALE_BLOCK_128  2  /* a_descale[M, ceil(K/128)], b_descale[ceil(N/128), ceil(K/128)] */

#define CF_EPI_NONE      0     /* C = bf16(acc * sa * sb)                          */
#define CF_EPI_BIAS      1     /* C = bf16(bf16(acc * sa * sb) + bias[n]), i.e. the GEMM followed by
                                  bias_add_strided_bf16 (kernels/moe.cu:325-334)   */
#define CF_EPI_SILU_GATE 2     /* C = swiglu(bf16(gate), bf16(up)): two weight matrices, the GEMMs at
                                  src/trainer.cu:6310-6312 followed by swiglu_forward (:6322) */

#define CF_GEMM_FLAG_NAIVE 1   /* run the one-lane-per-output cross-check kernel  */
#define CF_GEMM_FLAG_STAGED 2  /* take the register-staged tile kernel (the K % 64 != 0 path) */
#define CF_GEMM_FLAG_DUO 4     /* take the 128 x 128-tile kernel that runs two workgroups per CU (a tile's epilogue under
                                  the other workgroup's MFMAs) where it applies: E4M3, CF_SCALE_ROW_COL, plain or SiLU-gate
                                  epilogue, N a multiple of 128 (64 with the SiLU gate) */
#define CF_GEMM_FLAG_DUO_IN_STEP 8 /* with CF_GEMM_FLAG_DUO: do not start the CU's second workgroup half a tile late */
#define CF_GEMM_FLAG_MFMA32 16 /* plain, bias and SiLU-gate epilogues: keep the ring kernel on v_mfma_f32_32x32x64_f8f6f4
                                  instead of the one on v_mfma_f32_16x16x128_f8f6f4 (the default; same tiles and drain,
                                  8 - 9 % more MFMA throughput at the same socket power) */

/* lt_gemm_fp8_nt, static at src/trainer.cu:4498-4534 (plan lookup :4402-4496).
 * C[M,N] bf16 (row stride ldc) = (A[M,K] fp8, row stride lda, E4M3 or E5M2) .
 * (B[N,K] E4M3, contiguous)^T, per-tensor device descales, alpha 1, beta 0. */
int cf_fp8_gemm_nt_bf16(int M, int N, int K, const void* d_A, int lda, int a_is_e5m2,
                        const float* d_a_descale, const void* d_B, const float* d_b_descale,
                        uint16_t* d_C, int ldc, cf_stream_t stream);

/* Extended form of the same GEMM for the scale groups and fused epilogues of
 * the benchmark configurations (the reference runs src/trainer.cu:4498 and
 * then kernels/activations.cu:76-87 or kernels/moe.cu:349-356 as separate
 * launches).  d_bias is bf16 [N] for CF_EPI_BIAS; d_B_up / d_b_up_descale are
 * the second ("up") weight matrix [N,K] and its descale for CF_EPI_SILU_GATE;
 * unused pointers may be null. */
int cf_fp8_gemm_nt_bf16_ex(int M, int N, int K, const void* d_A, int lda, int a_is_e5m2,
                           const float* d_a_descale, const void* d_B, int ldb,
                           const float* d_b_descale, int scale_mode, int epilogue,
                           const uint16_t* d_bias, const void* d_B_up,
                           const float* d_b_up_descale, uint16_t* d_C, int ldc, int flags,
                           cf_stream_t stream);

/* lt_gemm_fp8_tn_accum_f32, fp32 overload, static at src/trainer.cu:4596-4627 (plan :4539-4594).
 * dW[M,N] fp32 (row stride ldc_dw) += (X^T[M,K] E4M3 * ds_x) . (dY^T[N,K] E5M2 * ds_dy)^T,
 * both operands contiguous with K innermost (pre-transposed), alpha 1, beta 1. */
int cf_fp8_gemm_tn_accum_f32(int M, int N, int K, const void* d_Xt_e4m3, const float* d_ds_x,
                             const void* d_dYt_e5m2, const float* d_ds_dy, float* d_dW,
                             int ldc_dw, cf_stream_t stream);
/* lt_gemm_fp8_tn_accum_f32, bf16 overload, static at src/trainer.cu:4670-4691. */
int cf_fp8_gemm_tn_accum_bf16(int M, int N, int K, const void* d_Xt_e4m3, const float* d_ds_x,
                              const void* d_dYt_e5m2, const float* d_ds_dy, uint16_t* d_dW,
                              int ldc_dw, cf_stream_t stream);
/* The accumulate GEMM of src/trainer.cu:4596-4627 with free operand formats and row strides, and
 * CF_GEMM_FLAG_NAIVE for the cross-check kernel; used by the tests and for fp32 inspection of
 * the accumulators. */
int cf_fp8_gemm_nt_accum_f32_ex(int M, int N, int K, const void* d_A, int lda, int a_is_e5m2,
                                const float* d_a_descale, const void* d_B, int ldb, int b_is_e5m2,
                                const float* d_b_descale, float* d_C, int ldc, int flags,
                                cf_stream_t stream);

/* ---- MoE routing and dispatch: kernels/moe.cu, kernels/cross_entropy.cu --------
 * Routing results are reproducible bit for bit: fixed reduction order, a
 * deterministic expf, ties broken towards the lowest expert index, row lists in
 * ascending row order (the reference fills them in atomicAdd arrival order,
 * kernels/moe.cu:576-577, so its lists equal these as sets). */

/* softmax_inplace_f32, kernels.hpp:193, kernels/cross_entropy.cu:193-197. */
int cf_softmax_inplace_f32(float* d_x, int rows, int cols, cf_stream_t stream);

/* moe_topk_route_f32, kernels.hpp:313-317, kernels/moe.cu:409-422: softmax, keep the
 * top_k probabilities per row (strict >, lowest index wins ties), zero the rest,
 * optionally renormalise the kept ones to sum 1.  The save pointers may be null.
 * The reference's kept[32] flag array (kernels/moe.cu:383) limits it to 32 experts;
 * this entry point takes up to 2048. */
int cf_moe_topk_route_f32(float* d_scores, int rows, int num_experts, int top_k,
                          cf_stream_t stream, float* d_row_sum_save, float* d_scores_save,
                          int normalize_topk);

/* moe_build_expert_row_lists, kernels.hpp:361-364, kernels/moe.cu:702-710.
 * counts[E]; row_indices[E, rows] expert-major, first counts[e] entries valid. */
int cf_moe_build_expert_row_lists(const float* d_route_weights, int* d_counts,
                                  int* d_row_indices, int rows, int num_experts,
                                  cf_stream_t stream);

/* moe_expert_offsets_from_counts, kernels.hpp:397-399, kernels/moe.cu:859-863. */
int cf_moe_expert_offsets_from_counts(const int* d_counts, int* d_offsets, int num_experts,
                                      cf_stream_t stream);

/* moe_gather_rows_u8 / moe_gather_rows_bf16, kernels.hpp:365-372, kernels/moe.cu:712-728.
 * width is in elements. */
int cf_moe_gather_rows_u8(const uint8_t* d_src, uint8_t* d_dst, const int* d_row_indices,
                          int n_rows, int width, cf_stream_t stream);
int cf_moe_gather_rows_bf16(const uint16_t* d_src, uint16_t* d_dst, const int* d_row_indices,
                            int n_rows, int width, cf_stream_t stream);

/* moe_scatter_accumulate_rows_bf16, kernels.hpp:373-377, kernels/moe.cu:730-738:
 * mixed[row_indices[i], h] = bf16(mixed + w[row, expert_idx] * compact[i, h]). */
int cf_moe_scatter_accumulate_rows_bf16(uint16_t* d_mixed, const uint16_t* d_compact,
                                        const float* d_route_weights, const int* d_row_indices,
                                        int n_rows, int expert_idx, int num_experts, int H,
                                        cf_stream_t stream);
/* moe_scale_accumulate_bf16, kernels.hpp:340-343, kernels/moe.cu:677-683 (dense form). */
int cf_moe_scale_accumulate_bf16(uint16_t* d_mixed, const uint16_t* d_term,
                                 const float* d_route_weights, int rows, int expert_idx,
                                 int num_experts, int H, cf_stream_t stream);

/* ---- grouped (per-expert) FP8 GEMM and the SwiGLU expert bank --------------------
 * The reference runs its selected-row expert path as a host loop of variable-M
 * cuBLASLt GEMMs after copying the counts to the host (src/trainer.cu:6876-6934), or as
 * one scalar-FMA kernel per (expert, row tile) (kernels/moe.cu:950-1127).  These entry
 * points keep the counts on the device and run every expert's tiles in one MFMA launch. */

/* Bytes of the tile table cf_fp8_grouped_gemm_nt_bf16_ex needs in d_workspace.  The reference's GEMM
 * workspace is the 32 MiB block owned by Fp8Ctx (src/trainer.cu:3300-3301); here the caller owns it. */
int cf_fp8_grouped_gemm_workspace_bytes(int total_rows, int num_experts, size_t* bytes);

/* For each expert e: C[offsets[e] .. +counts[e], :] = A_rows . B[e]^T with the per-token x
 * per-channel scales and epilogues of cf_fp8_gemm_nt_bf16_ex (replaces the per-expert
 * lt_gemm_fp8_nt calls at src/trainer.cu:6893-6931).  A row r of the compact output reads A row
 * d_a_row_index[r] (and its descale) when the index is given, so the token permute
 * (moe_gather_rows_u8, kernels/moe.cu:720-728) is fused into the operand fetch; null = row r.
 * B is [num_experts, N, K] E4M3, b_descale [num_experts, N].  total_rows is the host-side upper
 * bound rows * top_k; counts / offsets stay on the device.  a_rows is the number of rows of d_A
 * (every row index is below it; total_rows without an index).  Needs K % 128 == 0, K >= 256,
 * N a multiple of 8 (of 128 with the SiLU-gate epilogue), ldc % 8 == 0, 16-byte aligned operands,
 * descales and C, and a_rows * lda, N * K below 2^32. */
int cf_fp8_grouped_gemm_nt_bf16_ex(int total_rows, int N, int K, int num_experts,
                                   const int* d_counts, const int* d_offsets, const void* d_A,
                                   int a_rows, int lda, const int* d_a_row_index, const float* d_a_descale,
                                   const void* d_B, const float* d_b_descale, int scale_mode,
                                   int epilogue, const void* d_B_up, const float* d_b_up_descale,
                                   uint16_t* d_C, int ldc, void* d_workspace,
                                   size_t workspace_bytes, cf_stream_t stream);

/* cf_fp8_grouped_gemm_nt_bf16_ex for callers that cannot allocate device memory or own no workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments without the workspace, same kernels, same result bits; the tile table
 * lives in a fixed 64 KiB array inside the library's device image (one copy per GPU, held until the process
 * ends), so the call allocates nothing.  A shape whose table needs more than
 * cf_fp8_grouped_gemm_static_max_bytes() bytes (cf_fp8_grouped_gemm_workspace_bytes tells: more than
 * 3276 row tiles, total_rows / 256 + num_experts) returns CF_ERR_UNSUPPORTED and launches nothing.  Every
 * call on a GPU shares that GPU's array: calls that may overlap in time on one GPU (different streams,
 * different host threads) race on it and must be serialised by the caller; calls on one stream are ordered.
 * cf_fp8_grouped_gemm_static_max_bytes is also the set-up call: it looks up the array's address on the
 * current device, so a caller that will record the entry point into a graph calls it once per device first
 * (without it the first call of the entry point on a device does the lookup). */
int cf_fp8_grouped_gemm_static_max_bytes(size_t* bytes);
int cf_fp8_grouped_gemm_nt_bf16_static(int total_rows, int N, int K, int num_experts,
                                       const int* d_counts, const int* d_offsets, const void* d_A,
                                       int a_rows, int lda, const int* d_a_row_index, const float* d_a_descale,
                                       const void* d_B, const float* d_b_descale, int scale_mode,
                                       int epilogue, const void* d_B_up, const float* d_b_up_descale,
                                       uint16_t* d_C, int ldc, cf_stream_t stream);

/* ---- bf16 GEMMs of the selected-expert backward -------------------------------------
 * The reference's selected-expert backward runs, per expert and behind a host copy of the counts, four
 * cuBLAS calls on bf16 operands (src/trainer.cu:7727-7740; wrappers gemm_bf16 :3069-3090 and
 * gemm_bf16_tn_f32 :3116-3160, all with alpha = 1):
 *   d_act[n,Ie]   = d_expert_out[n,H] . fc_out_w[H,Ie]            gemm_bf16, beta = 0
 *   g_out[H,Ie]  += d_expert_out[n,H]^T . act[n,Ie]               gemm_bf16_tn_f32, beta = 1
 *   d_x[n,H]      = d_pre[n,Ie] . fc_in_w[Ie,H]                   gemm_bf16, beta = 0
 *   g_in[Ie,H]   += d_pre[n,Ie]^T . x[n,H]                        gemm_bf16_tn_f32, beta = 1
 * The dense forms below take the wrappers' arguments (row-major, row strides in elements); the grouped
 * forms run every expert in one launch over the forward's saved counts / offsets, the experts' rows
 * lying back to back in compact buffers (expert e owns rows offsets[e] .. offsets[e] + counts[e]).
 * fp32 accumulation on the matrix cores, one rounding to bf16.  Needs 16-byte aligned operands, row
 * strides that are multiples of 8 elements (C: of 4, below 2^21), N % 8 == 0, and K % 8 == 0 (nn) or
 * M % 8 == 0 (tn); the contraction length of the tn forms (an expert's row count) is arbitrary.
 * Shapes outside these return CF_ERR_UNSUPPORTED. */

/* C[M,N] = A[M,K] . B[K,N]   (gemm_bf16 with alpha = 1, beta = 0, src/trainer.cu:3069-3090) */
int cf_gemm_bf16_nn(int M, int N, int K, const uint16_t* d_A, int lda, const uint16_t* d_B, int ldb,
                    uint16_t* d_C, int ldc, cf_stream_t stream);
/* C[M,N] += A[K,M]^T . B[K,N]   (gemm_bf16_tn_f32 with alpha = 1, beta = 1; fp32 C, src/trainer.cu:3116-3137) */
int cf_gemm_bf16_tn_accum_f32(int M, int N, int K, const uint16_t* d_A, int lda, const uint16_t* d_B, int ldb,
                              float* d_C, int ldc, cf_stream_t stream);
/* the same with a bf16 C: bf16(float(C) + product), the overload at src/trainer.cu:3142-3160 */
int cf_gemm_bf16_tn_accum_bf16(int M, int N, int K, const uint16_t* d_A, int lda, const uint16_t* d_B, int ldb,
                               uint16_t* d_C, int ldc, cf_stream_t stream);
/* For each expert e: C[rows of e, :] = A[rows of e, :K] . B[e]  with B [num_experts, K, N] row-major
 * (the two input-gradient calls, src/trainer.cu:7729, 7738).  total_rows is the host-side bound rows * top_k;
 * d_workspace holds the tile table: cf_fp8_grouped_gemm_workspace_bytes(total_rows, num_experts) bytes. */
int cf_moe_grouped_gemm_bf16_nn(int total_rows, int N, int K, int num_experts, const int* d_counts,
                                const int* d_offsets, const uint16_t* d_A, int lda, const uint16_t* d_B,
                                uint16_t* d_C, int ldc, void* d_workspace, size_t workspace_bytes,
                                cf_stream_t stream);
/* For each expert e: C[e] += A[rows of e, :M]^T . B[rows of e, :N]  with C [num_experts, M, N]
 * (the two weight-gradient calls, src/trainer.cu:7727, 7736); an expert without rows leaves its C alone.
 * total_rows is the number of rows A and B hold: an expert's row range is cut there. */
int cf_moe_grouped_gemm_bf16_tn_accum_f32(int M, int N, int total_rows, int num_experts, const int* d_counts,
                                          const int* d_offsets, const uint16_t* d_A, int lda,
                                          const uint16_t* d_B, int ldb, float* d_C, cf_stream_t stream);
int cf_moe_grouped_gemm_bf16_tn_accum_bf16(int M, int N, int total_rows, int num_experts, const int* d_counts,
                                           const int* d_offsets, const uint16_t* d_A, int lda,
                                           const uint16_t* d_B, int ldb, uint16_t* d_C, cf_stream_t stream);

/* The selected-expert backward of the GELU expert bank (src/trainer.cu:7669-7741: per expert and behind the
 * host copy of the counts, the FP8 recompute of the forward, moe_row_dot_selected_bf16,
 * moe_gather_scale_rows_bf16, two gemm_bf16_tn_f32, two gemm_bf16, gelu_backward, moe_gather_rows_bf16 and
 * moe_scatter_add_rows_bf16) for every expert in one call with no host round trip, over the forward's saved
 * counts / offsets / row_indices.  Inputs: d_grad_mixed [rows,H] bf16; the FP8 hidden states [rows,H] with
 * their per-tensor descale and the bf16 hidden states [rows,H] (moe_hidden_gated); the dense route weights
 * [rows,E]; the expert weights as FP8 [E,Ie,H] / [E,H,Ie] with per-tensor descales (recompute) and as bf16
 * (gradients).  Outputs: d_grad_route_weights [rows,E] fp32 (cleared, then one entry per selected pair),
 * d_grad_fc_in [E,Ie,H] and d_grad_fc_out [E,H,Ie] bf16 (accumulated into), d_grad_hidden [rows,H] bf16
 * (accumulated into, experts in ascending order).  As in cf_moe_grouped_gelu_forward_fp8 the recomputed
 * activation is quantized with one scale per token row (cf_moe_grouped_gelu_backward_fp8_slots keeps the loop's
 * per-expert delayed scale).  H and Ie multiples of 128 and at least 256; total_selected_rows an upper bound on
 * the sum of the counts; d_workspace
 * 256-byte aligned.  cf_moe_grouped_gelu_backward_workspace gives the workspace size and, when `offsets` is
 * not null, the byte offsets of the intermediates inside it (CF_MOE_BWD_WS_* order), which stay valid after
 * the call: pre / post / postq / d_out / d_post / d_pre / x / d_x, experts back to back. */
enum {
    CF_MOE_BWD_WS_TILE_MAP = 0, CF_MOE_BWD_WS_INDEX, CF_MOE_BWD_WS_HIDDEN_DESCALE, CF_MOE_BWD_WS_IN_DESCALE,
    CF_MOE_BWD_WS_OUT_DESCALE, CF_MOE_BWD_WS_PRE, CF_MOE_BWD_WS_POST, CF_MOE_BWD_WS_POSTQ, CF_MOE_BWD_WS_POST_SCALE,
    CF_MOE_BWD_WS_POST_DESCALE, CF_MOE_BWD_WS_D_OUT, CF_MOE_BWD_WS_D_POST, CF_MOE_BWD_WS_D_PRE, CF_MOE_BWD_WS_X,
    CF_MOE_BWD_WS_D_X, CF_MOE_BWD_WS_COUNT
};
int cf_moe_grouped_gelu_backward_workspace(int rows, int total_selected_rows, int num_experts, int H, int Ie,
                                           size_t* offsets, size_t* bytes);
int cf_moe_grouped_gelu_backward_fp8(const uint16_t* d_grad_mixed, const void* d_hidden_fp8,
                                     const float* d_fcin_descale, int fcin_is_e5m2,
                                     const uint16_t* d_hidden_bf16, const float* d_route_weights,
                                     const int* d_counts, const int* d_offsets, const int* d_row_indices,
                                     const void* d_fc_in_w8, const float* d_fc_in_descale,
                                     const void* d_fc_out_w8, const float* d_fc_out_descale,
                                     const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w,
                                     float* d_grad_route_weights, uint16_t* d_grad_fc_in,
                                     uint16_t* d_grad_fc_out, uint16_t* d_grad_hidden, int rows, int H, int Ie,
                                     int num_experts, int total_selected_rows, void* d_workspace,
                                     size_t workspace_bytes, cf_stream_t stream);

/* Row lists of all experts back to back: compact[offsets[e] + s] = row_indices[e, s]
 * (the gather order of moe_gather_rows_u8 over all experts, kernels/moe.cu:594-606). */
int cf_moe_compact_row_index(const int* d_counts, const int* d_offsets, const int* d_row_indices,
                             int rows, int num_experts, int* d_compact_index, cf_stream_t stream);

/* All per-expert moe_scatter_accumulate_rows_bf16 launches (kernels/moe.cu:730-738,
 * src/trainer.cu:6932-6934) in one: experts in ascending order per token row, one bf16
 * rounding per expert.  compact_out is [sum counts, H] in compact-row order; the row lists
 * must be ascending (as cf_moe_build_expert_row_lists builds them). */
int cf_moe_unpermute_weighted_bf16(uint16_t* d_mixed, const uint16_t* d_compact_out,
                                   const float* d_route_weights, const int* d_counts,
                                   const int* d_offsets, const int* d_row_indices, int rows,
                                   int num_experts, int H, cf_stream_t stream);

/* ---- MoE expert-bank backward with the forward's routes (src/trainer.cu:7654-7741) --------
 * The custom kernels of the selected-expert backward; its bf16 GEMMs are BLAS calls in the
 * reference (gemm_bf16 / gemm_bf16_tn_f32) and stay BLAS calls. */

/* gelu_forward, kernels.hpp:334, kernels/moe.cu:510-521: out = bf16(0.5 x (1 + erf(x / sqrt 2))). */
int cf_gelu_forward_bf16(const uint16_t* d_x, uint16_t* d_out, size_t n, cf_stream_t stream);
/* gelu_backward, kernels/moe.cu:1148-1167: grad_pre = bf16(grad_post * (Phi(pre) + pre phi(pre))). */
int cf_gelu_backward_bf16(const uint16_t* d_pre, const uint16_t* d_grad_post, uint16_t* d_grad_pre,
                          size_t n, cf_stream_t stream);

/* moe_row_dot_selected_bf16, kernels/moe.cu:623-645,740-748:
 * out[row_indices[i] * out_stride + out_col] = dot(a_full[row_indices[i]], b_compact[i]), summed in the
 * reference's order (min(H, 256) strided partial sums, then a halving tree). */
int cf_moe_row_dot_selected_bf16(const uint16_t* d_a_full, const uint16_t* d_b_compact, float* d_out,
                                 const int* d_row_indices, int n_rows, int H, int out_stride,
                                 int out_col, cf_stream_t stream);
/* moe_gather_scale_rows_bf16, kernels/moe.cu:646-660,750-758:
 * dst[i, h] = bf16(w[row_indices[i], expert_idx] * src[row_indices[i], h]). */
int cf_moe_gather_scale_rows_bf16(const uint16_t* d_src, uint16_t* d_dst, const float* d_route_weights,
                                  const int* d_row_indices, int n_rows, int expert_idx,
                                  int num_experts, int H, cf_stream_t stream);
/* moe_scatter_add_rows_bf16, kernels/moe.cu:661-674,760-767:
 * dst_full[row_indices[i], h] = bf16(dst_full + src_compact[i, h]). */
int cf_moe_scatter_add_rows_bf16(uint16_t* d_dst_full, const uint16_t* d_src_compact,
                                 const int* d_row_indices, int n_rows, int H, cf_stream_t stream);

/* The two per-expert launches moe_row_dot_selected_bf16 + moe_gather_scale_rows_bf16 of every
 * expert (src/trainer.cu:7722-7725) in one launch over the forward's saved lists:
 *   grad_route_weights[row, e] = dot(grad_mixed[row], expert_out[slot])   (0 where e did not select row)
 *   expert_out[slot]           = bf16(route_weights[row, e] * grad_mixed[row])   (in place)
 * slot = offsets[e] + position of row in expert e's list; expert_out is [sum counts, H]. */
int cf_moe_grouped_route_grad_bf16(const uint16_t* d_grad_mixed, uint16_t* d_expert_out,
                                   float* d_grad_route_weights, const float* d_route_weights,
                                   const int* d_counts, const int* d_offsets, const int* d_row_indices,
                                   int rows, int num_experts, int H, cf_stream_t stream);
/* All per-expert moe_scatter_add_rows_bf16 launches (src/trainer.cu:7739-7740) in one: experts
 * in ascending order per token row, one bf16 rounding per expert; the route weights only mark
 * which experts selected a row.  Same layout rules as cf_moe_unpermute_weighted_bf16. */
int cf_moe_unpermute_add_bf16(uint16_t* d_dst_full, const uint16_t* d_src_compact,
                              const float* d_route_weights, const int* d_counts, const int* d_offsets,
                              const int* d_row_indices, int rows, int num_experts, int H,
                              cf_stream_t stream);

/* The unpermute without the search: cf_moe_build_slot_index writes
 * slot_index[row, e] = offsets[e] + position of row in expert e's list for every listed pair
 * ([rows, num_experts] ints; other cells are not touched and not read), once per routing;
 * cf_moe_unpermute_indexed_bf16 is then cf_moe_unpermute_weighted_bf16 (unit_weights = 0,
 * kernels/moe.cu:730-738) or cf_moe_unpermute_add_bf16 (unit_weights = 1, kernels/moe.cu:760-767)
 * with the same results.  No ordering requirement on the lists. */
int cf_moe_build_slot_index(const int* d_counts, const int* d_offsets, const int* d_row_indices,
                            int rows, int num_experts, int* d_slot_index, cf_stream_t stream);
int cf_moe_unpermute_indexed_bf16(uint16_t* d_mixed, const uint16_t* d_compact_out,
                                  const float* d_route_weights, const int* d_slot_index, int rows,
                                  int num_experts, int H, int unit_weights, cf_stream_t stream);

/* The grouped SwiGLU expert bank of benchmark config 5 (the FP8 form of the expert loop in
 * moe_expert_bank_forward, src/trainer.cu:6876-6934, with the SwiGLU experts of
 * moe_generic_forward, src/trainer.cu:6510-6529): permute -> gate/up GEMM with fused SiLU gate
 * -> per-token E4M3 quantize -> down GEMM -> weighted unpermute added into d_mixed.
 * hidden [rows,H] E4M3 with per-token descales; w_gate / w_up [E,Ie,H], w_down [E,H,Ie] E4M3 with
 * per-channel descales [E,Ie] / [E,H].  d_workspace: 256-byte aligned,
 * cf_moe_grouped_swiglu_workspace_bytes() bytes. */
int cf_moe_grouped_swiglu_workspace_bytes(int total_selected_rows, int num_experts, int H,
                                          int Ie, size_t* bytes);
int cf_moe_grouped_swiglu_forward_fp8(const void* d_hidden_e4m3, const float* d_hidden_descale,
                                      const float* d_route_weights, const int* d_counts,
                                      const int* d_offsets, const int* d_row_indices,
                                      const void* d_w_gate, const float* d_w_gate_descale,
                                      const void* d_w_up, const float* d_w_up_descale,
                                      const void* d_w_down, const float* d_w_down_descale,
                                      uint16_t* d_mixed, int rows, int H, int Ie, int num_experts,
                                      int total_selected_rows, void* d_workspace,
                                      size_t workspace_bytes, cf_stream_t stream);

/* moe_grouped_expert_forward_fp8, kernels.hpp:400-423, kernels/moe.cu:1063-1127 (kernel :950-1060):
 * mixed[row] += w[row,e] * fc_out_e(gelu(fc_in_e(hidden[row]))) for every selected (expert,row);
 * per-tensor device descales, exact-erf GELU kept in fp32 (not re-quantised), bf16 accumulation
 * by compare-and-swap, so the last bit of d_mixed depends on arrival order as in the reference.
 * fc_in_w [E,Ie,H], fc_out_w [E,H,Ie] E4M3; hidden E4M3 or E5M2.  d_offsets and
 * total_selected_rows are accepted and unused, as in the reference.  With H % 128 == 0,
 * Ie % 64 == 0, 16-byte aligned operands and 8-byte aligned d_mixed the two projections run on
 * the matrix cores (fp8 MFMA for fc_in; fc_out as bf16 MFMA on a two-term bf16 split of the fp32
 * GELU output, relative error 2^-17, against the weights widened exactly; 32 token rows per
 * workgroup up to H = 2048, 16 beyond); other shapes take a wave-parallel fp32 kernel.  Same contract
 * either way. */
int cf_moe_grouped_expert_forward_fp8(const void* d_hidden, const float* d_fcin_descale,
                                      int fcin_is_e5m2, const float* d_route_weights,
                                      const int* d_counts, const int* d_offsets,
                                      const int* d_row_indices, const void* d_fc_in_w,
                                      const float* d_fc_in_descale, const void* d_fc_out_w,
                                      const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                      int H, int Ie, int num_experts, int total_selected_rows,
                                      cf_stream_t stream);

/* moe_grouped_expert_forward_fp8 (kernels.hpp:400-423, kernels/moe.cu:950-1127) with a workspace: the same
 * arguments and contract as cf_moe_grouped_expert_forward_fp8, run as whole-matrix launches when H % 128 == 0,
 * H >= 256, Ie % 128 == 0, Ie <= 4096 and hidden, weights and d_mixed are 16-byte aligned (other shapes are
 * passed on to that function and need no workspace).  fc_in is one grouped FP8 GEMM over the gathered token
 * rows with fp32 output; the GELU is taken in fp32 (erf to 1.5e-7 absolute) and each row is written as three
 * E4M3 terms under one per-row scale (value * scale = q0 + q1 / 16 + q2 / 256 to 2^-13: 12 to 13 significand
 * bits, not re-quantized to a single fp8 value); fc_out is one grouped FP8 GEMM over K = 3 Ie in which the
 * matrix cores weight term t by 2^(-4 t) (E8M0 scales of the MX form of the FP8 MFMA), so the three partial
 * products add in one fp32 accumulator and y stays fp32; w * y is then added into d_mixed per token row over its
 * experts in ascending order, one bf16 rounding per expert as in the reference's compare-and-swap add.  The
 * one difference from the reference kernel: the order of the adds is fixed.  total_selected_rows is an upper bound on
 * the sum of d_counts (rows * top_k, as the reference's caller passes it); d_offsets may be null (the offsets are recomputed).
 * The workspace belongs to the call: two calls that may overlap in time (two streams, two host threads) need two workspaces.
 * d_workspace 256-byte aligned; cf_moe_grouped_expert_forward_fp8_workspace gives its size and, when
 * `offsets` is not null, the byte offsets of the intermediates (CF_MOE_FWD_WS_* order), which stay valid
 * after the call: pre [total, Ie] fp32, split [total, 3 Ie] E4M3, split_descale [total] fp32, y [total, H] fp32,
 * experts back to back (CF_MOE_FWD_WS_X is reserved and has no bytes). */
enum {
    CF_MOE_FWD_WS_TILE_MAP = 0, CF_MOE_FWD_WS_OFFSETS, CF_MOE_FWD_WS_INDEX, CF_MOE_FWD_WS_SLOT, CF_MOE_FWD_WS_PRE,
    CF_MOE_FWD_WS_SPLIT, CF_MOE_FWD_WS_SPLIT_DESCALE, CF_MOE_FWD_WS_Y, CF_MOE_FWD_WS_X, CF_MOE_FWD_WS_COUNT
};
int cf_moe_grouped_expert_forward_fp8_workspace(int rows, int total_selected_rows, int num_experts, int H,
                                                int Ie, size_t* offsets, size_t* bytes);
int cf_moe_grouped_expert_forward_fp8_ws(const void* d_hidden, const float* d_fcin_descale,
                                         int fcin_is_e5m2, const float* d_route_weights,
                                         const int* d_counts, const int* d_offsets,
                                         const int* d_row_indices, const void* d_fc_in_w,
                                         const float* d_fc_in_descale, const void* d_fc_out_w,
                                         const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                         int H, int Ie, int num_experts, int total_selected_rows,
                                         void* d_workspace, size_t workspace_bytes, cf_stream_t stream);

/* moe_grouped_expert_forward_bf16 (kernels.hpp:400-407, kernels/moe.cu:800-851) with a workspace: the same
 * arguments and contract as cf_moe_grouped_expert_forward_bf16, run as whole-matrix launches when H % 8 == 0,
 * Ie % 64 == 0 and the operands are 16-byte aligned (other shapes are passed on to that function).  fc_in is one
 * grouped bf16 GEMM that gathers the selected token rows in its operand fetch, fp32 output (pre); the GELU (fp32,
 * erf to 1.5e-7 absolute) is rounded to bf16 as the reference kernel rounds it before fc_out (split [total, Ie]
 * bf16); fc_out is one grouped bf16 GEMM, fp32 out (y); then the ordered add into d_mixed as in
 * cf_moe_grouped_expert_forward_fp8_ws, with the same one difference from the reference kernel.  Workspace rules
 * as there; CF_MOE_FWD_WS_SPLIT_DESCALE is unused. */
int cf_moe_grouped_expert_forward_bf16_workspace(int rows, int total_selected_rows, int num_experts, int H,
                                                 int Ie, size_t* offsets, size_t* bytes);
int cf_moe_grouped_expert_forward_bf16_ws(const uint16_t* d_hidden, const float* d_route_weights,
                                          const int* d_counts, const int* d_offsets,
                                          const int* d_row_indices, const uint16_t* d_fc_in_w,
                                          const uint16_t* d_fc_out_w, uint16_t* d_mixed, int rows, int H,
                                          int Ie, int num_experts, int total_selected_rows,
                                          void* d_workspace, size_t workspace_bytes, cf_stream_t stream);

/* moe_grouped_expert_forward_bf16, kernels.hpp:400-407 (kernel kernels/moe.cu:800-851): the same
 * device-scheduled expert bank on bf16 hidden states and bf16 weights (fc_in_w [E,Ie,H], fc_out_w
 * [E,H,Ie]), no descales; fp32 accumulation, exact-erf GELU rounded to bf16 before fc_out (as the
 * kernel's shared-memory row holds it, :845), compare-and-swap accumulation into d_mixed.  The
 * non-FP8 sibling: bf16 MFMA for both projections when H % 64 == 0, Ie % 64 == 0, the operands are
 * 16-byte aligned and d_mixed 8-byte aligned (16-row tiles); a wave-parallel fp32 kernel
 * otherwise. */
int cf_moe_grouped_expert_forward_bf16(const uint16_t* d_hidden, const float* d_route_weights,
                                       const int* d_counts, const int* d_offsets,
                                       const int* d_row_indices, const uint16_t* d_fc_in_w,
                                       const uint16_t* d_fc_out_w, uint16_t* d_mixed, int rows,
                                       int H, int Ie, int num_experts, int total_selected_rows,
                                       cf_stream_t stream);

/* gelu_forward (kernels/moe.cu:510-521) followed by the per-token E4M3 quantize of its bf16
 * output, in one pass: out = e4m3(bf16(gelu(x)) * scale[row]), scale[row] = 448 / max(amax, 1e-12)
 * over the row of bf16(gelu(x)), descale its inverse (the formula of kernels/fp8.cu:37-39,49).
 * Bytes and scales equal cf_gelu_forward_bf16 then cf_fp8_quantize_rows. */
int cf_gelu_quantize_rows_e4m3(const uint16_t* d_x, int rows, int K, void* d_out, float* d_scale,
                               float* d_descale, cf_stream_t stream);

/* The FP8 expert loop of moe_expert_bank_forward (src/trainer.cu:6886-6934: moe_gather_rows_u8 ->
 * lt_gemm_fp8_nt fc_in -> gelu_forward -> quantize -> lt_gemm_fp8_nt fc_out ->
 * moe_scatter_accumulate_rows_bf16, once per expert behind a host synchronisation) for every expert
 * in one call with no host round trip, on the FP8 matrix cores: same arguments as
 * cf_moe_grouped_expert_forward_fp8 plus a workspace.  Unlike that function (and like the loop)
 * the GELU output is rounded to bf16 and re-quantized to E4M3 before fc_out; its scale is per
 * token row; cf_moe_grouped_gelu_forward_fp8_slots below keeps the loop's per-expert delayed scale
 * instead.  d_offsets must be the exclusive prefix sum of d_counts, total_selected_rows an upper
 * bound on their sum.  H and Ie multiples of 128 and at least 256; d_workspace 256-byte aligned,
 * cf_moe_grouped_gelu_workspace_bytes() bytes. */
int cf_moe_grouped_gelu_workspace_bytes(int rows, int total_selected_rows, int num_experts, int H,
                                        int Ie, size_t* bytes);
int cf_moe_grouped_gelu_forward_fp8(const void* d_hidden, const float* d_fcin_descale,
                                    int fcin_is_e5m2, const float* d_route_weights,
                                    const int* d_counts, const int* d_offsets,
                                    const int* d_row_indices, const void* d_fc_in_w,
                                    const float* d_fc_in_descale, const void* d_fc_out_w,
                                    const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                    int H, int Ie, int num_experts, int total_selected_rows,
                                    void* d_workspace, size_t workspace_bytes, cf_stream_t stream);

/* The steady-state branch of fp8_quant_act (src/trainer.cu:4823-4850) for a bank of per-expert activation slots in ONE
 * launch: what the FP8 expert loop does once per expert on moe_fcout_act_slot(f8, layer, base + e) between its two
 * GEMMs (src/trainer.cu:6910-6918).  d_x [total_rows, K] bf16 holds the experts' rows back to back (expert e:
 * d_counts[e] rows from row d_offsets[e]); block e of d_slot_states (state_stride_words 4-byte words apart, each laid
 * out as the device block of a cf_act_slot with this history_len) is expert e's slot.  Per expert with at least one
 * row: the scale pair the previous call left is snapshotted, the rows are quantized with it (E4M3 or E5M2) while their
 * amax is recorded, and history, cursor, count, scale and descale advance as fp8_update_delayed_scale does; an
 * expert without rows keeps its state untouched, as the loop's `continue` leaves it (:6887-6888).  apply_gelu: the
 * tensor quantized is bf16(gelu(x)) (gelu_forward in place, kernels/moe.cu:510-521, then the quantize).
 * is_recompute: quantize with the snapshot scale and change nothing (:4736-4743).  d_row_descale [total_rows]
 * receives, for every row, its expert's descale_snapshot: what the GEMM consuming the bytes dequantizes with
 * (:6921-6924).  The slots must be in steady state (calibration and first use go through cf_fp8_quant_act per
 * expert) and share one format.  K % 16 == 0, 16-byte aligned d_x and d_out.  Calls on one bank must not overlap. */
int cf_moe_grouped_quantize_delayed(const uint16_t* d_x, void* d_out, int K, int num_experts,
                                    const int* d_counts, const int* d_offsets, int total_rows,
                                    float* d_slot_states, int state_stride_words, int history_len,
                                    int is_e5m2, int apply_gelu, int is_recompute, float* d_row_descale,
                                    cf_stream_t stream);

/* cf_moe_grouped_gelu_forward_fp8 with the reference loop's activation scale: the GELU output of expert e is
 * quantized by cf_moe_grouped_quantize_delayed on slot e of d_fcout_slot_states (fp8_quant_act on
 * moe_fcout_act_slot(..., e), src/trainer.cu:6916-6918) and fc_out dequantizes with that slot's descale_snapshot
 * (:6921-6924); fcout_is_e5m2 is act_fp8_type of those slots.  is_recompute replays a forward for the backward
 * (snapshot scale, no side effects).  Same workspace as cf_moe_grouped_gelu_forward_fp8. */
int cf_moe_grouped_gelu_forward_fp8_slots(const void* d_hidden, const float* d_fcin_descale,
                                          int fcin_is_e5m2, const float* d_route_weights,
                                          const int* d_counts, const int* d_offsets,
                                          const int* d_row_indices, const void* d_fc_in_w,
                                          const float* d_fc_in_descale, const void* d_fc_out_w,
                                          const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                          int H, int Ie, int num_experts, int total_selected_rows,
                                          float* d_fcout_slot_states, int state_stride_words,
                                          int history_len, int fcout_is_e5m2, int is_recompute,
                                          void* d_workspace, size_t workspace_bytes, cf_stream_t stream);

/* cf_moe_grouped_gelu_backward_fp8 whose recompute quantizes the GELU output as the reference's backward loop does:
 * fp8_quant_act with is_recompute = true on the expert's slot (src/trainer.cu:7707-7712), i.e. with the scale the
 * forward call snapshotted and no side effects.  Same workspace as cf_moe_grouped_gelu_backward_fp8. */
int cf_moe_grouped_gelu_backward_fp8_slots(const uint16_t* d_grad_mixed, const void* d_hidden_fp8,
                                           const float* d_fcin_descale, int fcin_is_e5m2,
                                           const uint16_t* d_hidden_bf16, const float* d_route_weights,
                                           const int* d_counts, const int* d_offsets, const int* d_row_indices,
                                           const void* d_fc_in_w8, const float* d_fc_in_descale,
                                           const void* d_fc_out_w8, const float* d_fc_out_descale,
                                           const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w,
                                           float* d_grad_route_weights, uint16_t* d_grad_fc_in,
                                           uint16_t* d_grad_fc_out, uint16_t* d_grad_hidden, int rows, int H, int Ie,
                                           int num_experts, int total_selected_rows,
                                           float* d_fcout_slot_states, int state_stride_words, int history_len,
                                           int fcout_is_e5m2, void* d_workspace, size_t workspace_bytes,
                                           cf_stream_t stream);

/* A measuring stick for the benchmark, with no counterpart in the reference and no part in the hot path: a kernel
 * with the memory traffic of the per-token quantize (per row 2 x row_bytes_out bytes read, row_bytes_out written with
 * the same streaming stores, one wavefront per row) and next to no arithmetic.  row_bytes_out % 1024 == 0. */
int cf_hbm_stream_probe_2r1w(const void* d_src, void* d_dst, int rows, int row_bytes_out, cf_stream_t stream);

/* ---- slot state machines (host logic of src/trainer.cu over the entry points above) ------- */

/* One delayed-scaling activation / gradient call site: ActSlot, src/trainer.cu:3247-3279.  The host
 * object holds the flags (init, calib_remaining, calib_commit_pending, fp8_max); the device scalars
 * (amax, scale, descale, the two snapshots, calib min/max, cursor, count, history) live in one
 * caller-owned device block of cf_act_slot_state_words(history_len) 4-byte words. */
typedef struct cf_act_slot cf_act_slot;

/* words of device state one slot needs (alloc_act_slot, src/trainer.cu:4176-4201, allocates the same scalars) */
int cf_act_slot_state_words(int history_len);

/* alloc_act_slot, src/trainer.cu:4176-4201: history, cursor, count zeroed, calib_min = 0x7f7f7f7f,
 * calib_max = 0.  history_len is kActHistoryLen (8, src/trainer.cu:3213) in the reference and 16 in
 * benchmark config 3; calib_calls is IDA_FP8_CALIB_CALLS (default 8, src/trainer.cu:3765-3774),
 * type_spread_threshold is IDA_FP8_TYPE_SPREAD (default 4, src/trainer.cu:3778-3787). */
int cf_act_slot_create(cf_act_slot** out, void* d_state, int history_len, float fp8_max,
                       int calib_calls, float type_spread_threshold, cf_stream_t stream);
int cf_act_slot_destroy(cf_act_slot* slot);   /* frees the host object (src/trainer.cu:4176: slots die with the arena) */

/* act_fp8_type, src/trainer.cu:4728-4730: 1 when the slot writes E5M2 */
int cf_act_slot_is_e5m2(const cf_act_slot* slot);

#define CF_SLOT_AMAX 0
#define CF_SLOT_SCALE 1
#define CF_SLOT_DESCALE 2
#define CF_SLOT_SCALE_SNAPSHOT 3
#define CF_SLOT_DESCALE_SNAPSHOT 4   /* what the GEMM consuming the quantized tensor dequantizes with, src/trainer.cu:6118-6122 */
#define CF_SLOT_HISTORY 5
#define CF_SLOT_CURSOR 6
#define CF_SLOT_COUNT 7
#define CF_SLOT_CALIB_MIN 8
#define CF_SLOT_CALIB_MAX 9
/* device address of one of the slot's scalars (the ActSlot members of src/trainer.cu:3248-3278) */
int cf_act_slot_device_field(const cf_act_slot* slot, int field, void** d_ptr);

/* fp8_quant_act, src/trainer.cu:4732-4851: recompute (snapshot scale, no side effects); pending
 * calibration commit (host sync, may switch the slot to E5M2); calibration and first use (exact amax);
 * steady state (previous scale, record amax, advance the history).  The clip-debug probes of
 * src/trainer.cu:4834-4839 are separate entry points here. */
int cf_fp8_quant_act(cf_act_slot* slot, const uint16_t* d_x, void* d_act8, size_t n,
                     int is_recompute, cf_stream_t stream);

/* One Fp8Slot of refresh_fp8_weights, src/trainer.cu:4694-4712: (optional amax) -> scale -> fwd8 [out,in]
 * and bwd8 [in,out], one by direct quantize and one by quantize-transpose depending on how w is stored. */
int cf_fp8_refresh_weight(const uint16_t* d_w, void* d_fwd8, void* d_bwd8, float* d_amax,
                          float* d_scale, float* d_descale, int in_dim, int out_dim,
                          int stored_out_major, int recompute_amax, cf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CF_FP8_H */
