/*
 * cf_oracle.h -- CPU restatement of the reference FP8 hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing here is part of the shipped library: the
 * only permitted users are the test suite, the smoke check and the
 * cpu_baseline leg of the benchmark.  The HIP library never links, loads or
 * calls this code and has no CPU fallback.
 *
 * Every function cites the reference file:line whose arithmetic it restates
 * (paths relative to the reference tree root).  Compile with
 * -ffp-contract=off: the reference semantics are separate IEEE fp32
 * multiplies / divides, never fused.
 *
 * Pinning status (what independently fixes each function's answers):
 *   orc_e4m3_pack / unpack        reference header compiled on the host
 *                                 (oracle/_ref), exhaustive bf16 x scales and a
 *                                 strided fp32 sweep; probe bytes from
 *                                 tests/fp8_e4m3_probe.cu:23-27,55-56;
 *                                 torch.float8_e4m3fn cast after clamping.
 *   orc_e4m3_satfinite            same as pack for finite input; +-inf -> +-448
 *                                 from the reference comment kernels/fp8.cu:333-337.
 *                                 NaN payload: parity unpinned (needs nvcc).
 *   orc_e5m2_satfinite / unpack   OCP closed form, brute force against
 *                                 nearest-value search over all 256 codes and
 *                                 torch.float8_e5m2 after clamping.  The
 *                                 reference holds no test for E5M2:
 *                                 parity unpinned by the reference itself.
 *   amax / scale / delayed scale  closed forms + brute-force sequences.
 *   transposes / gathers          permutation identities on ragged shapes.
 *   softmax / top-k               tests/fixtures/moe_router_parity (JSON),
 *                                 invariants, brute force on tiny E.
 *   grouped GELU expert bank      the reference's router-parity fixture also holds
 *                                 hidden_gated / route_weights / weights / mixed:
 *                                 formula reproduced in float64 to 4e-8, FP8 form
 *                                 to quantization error (tests/golden/moe_expert_bank.json).
 *   orc_expf                      <= 2 ulp of the double-precision exp over a
 *                                 dense sweep (it is this build's definition of
 *                                 the router's expf; CUDA's expf bits cannot be
 *                                 obtained here: parity unpinned beyond ulp level).
 *   rmsnorm / row clip            see cf_oracle_norm.c (closed forms, double
 *                                 recomputation, order-sensitive crafted row;
 *                                 summation order beyond the source text:
 *                                 parity unpinned).
 *   cross-entropy                 see cf_oracle_ce.c (closed forms, sum-to-zero,
 *                                 double recomputation; libm exp/log stand in
 *                                 for CUDA's: parity unpinned beyond 1 bf16 ulp).
 *   MoE backward helpers          see cf_oracle_moe_bwd.c (exact-product row dot
 *                                 with the reference's summation tree, closed
 *                                 forms; libm erff / expf stand in for CUDA's in
 *                                 the GELU pair: parity unpinned beyond 1 bf16 ulp).
 *   swiglu backward               grad_up must equal the forward applied to
 *                                 (gate, grad_out) bit for bit (one commutative
 *                                 product); grad_gate against the closed form in
 *                                 double and a central difference; orc_expf
 *                                 stands in for CUDA's expf, as in the forward:
 *                                 parity unpinned beyond 1 bf16 ulp.
 *   column sum (bias gradient)    exactly summable integers against numpy; a
 *                                 column (2^24, then ones) whose sequential sum
 *                                 differs from every tree.
 *   bf16 GEMMs of the MoE backward (tests/oracle_lib.py: gemm_bf16_*_ref) double
 *                                 matmul of the same bf16 operands; exact-integer
 *                                 cases bit for bit.  cuBLAS's accumulation order:
 *                                 parity unpinned.
 *   GEMM references               definition from the task statement: matmul
 *                                 of the dequantised operands; special cases
 *                                 reduce to numpy matmul.  cuBLASLt's own
 *                                 accumulation order: parity unpinned.
 */
#ifndef CF_ORACLE_H
#define CF_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_E4M3_MAX 448.0f
#define ORC_E5M2_MAX 57344.0f

/* ---- scalar conversions ------------------------------------------------ */
uint16_t orc_bf16_from_f32(float v);
float    orc_bf16_to_f32(uint16_t b);
uint8_t  orc_e4m3_pack(float v, int* finite);
float    orc_e4m3_unpack(uint8_t b);
uint8_t  orc_e4m3_satfinite(float v);
uint8_t  orc_e5m2_satfinite(float v);
float    orc_e5m2_unpack(uint8_t b);
float    orc_expf(float x);

/* vector helpers for the tests (n elements each) */
void orc_bf16_from_f32_n(const float* in, uint16_t* out, size_t n);
void orc_bf16_to_f32_n(const uint16_t* in, float* out, size_t n);
void orc_e4m3_pack_n(const float* in, uint8_t* out, uint8_t* finite, size_t n);
void orc_e4m3_satfinite_n(const float* in, uint8_t* out, size_t n);
void orc_e5m2_satfinite_n(const float* in, uint8_t* out, size_t n);
void orc_e4m3_unpack_n(const uint8_t* in, float* out, size_t n);
void orc_e5m2_unpack_n(const uint8_t* in, float* out, size_t n);
void orc_expf_n(const float* in, float* out, size_t n);

/* ---- per-tensor quantize family (kernels/fp8.cu) ------------------------ */
void orc_amax_bf16(const uint16_t* x, size_t n, float* amax);
void orc_scale_from_amax(const float* amax, float fp8_max, float* scale, float* descale);
void orc_quantize_e4m3(const uint16_t* x, uint8_t* out, const float* scale, size_t n);
void orc_quantize_e5m2(const uint16_t* x, uint8_t* out, const float* scale, size_t n);
void orc_quantize_e4m3_record(const uint16_t* x, uint8_t* out, const float* scale, float* amax, size_t n);
void orc_quantize_e5m2_record(const uint16_t* x, uint8_t* out, const float* scale, float* amax, size_t n);
void orc_update_delayed_scale(const float* amax, float fp8_max, float* scale, float* descale,
                              float* history, int history_len, int* cursor, int* count);
void orc_quantize_transpose_e4m3(const uint16_t* w, uint8_t* out, const float* scale, int K, int N);
void orc_quant_and_transpose_e4m3(const uint16_t* in, uint8_t* act8, uint8_t* snap,
                                  const float* scale, int K, int N);
void orc_transpose_u8(const uint8_t* in, uint8_t* out, int rows, int cols);
void orc_clip_probe(const float* amax, const float* scale, float fp8_max, float* stats);
void orc_elem_clip_count(const uint16_t* x, const float* scale, float fp8_max, size_t n, float* out);
void orc_pack_bf16_e4m3_raw(const uint16_t* x, uint8_t* out, float* amax, float* scale,
                            float* descale, int* bad_count, size_t n);
void orc_pack_bf16_e4m3_raw_and_dequant(const uint16_t* x, uint8_t* out, uint16_t* dequant,
                                        float* amax, float* scale, float* descale,
                                        int* bad_count, size_t n);
void orc_unpack_e4m3_raw_bf16(const uint8_t* in, const float* descale, uint16_t* out, size_t n);
void orc_calib_minmax_update(const float* amax, float* cmin, float* cmax);

/* ---- scale-group extensions (same scale formula, smaller groups) -------- */
/* fp32 input, per-tensor (benchmark config 1) */
void orc_amax_f32(const float* x, size_t n, float* amax);
void orc_quantize_f32_e4m3(const float* x, uint8_t* out, const float* scale, size_t n);
/* one scale per row of x[rows,K] */
void orc_quantize_rows(const uint16_t* x, int rows, int K, int is_e5m2,
                       uint8_t* out, float* scale, float* descale);
/* one scale per 1 x 128 group along K; scales laid out [rows, ceil(K/128)] */
void orc_quantize_block_1x128(const uint16_t* x, int rows, int K,
                              uint8_t* out, float* scale, float* descale);
/* one scale per 128 x 128 block; scales laid out [ceil(rows/128), ceil(K/128)] */
void orc_quantize_block_128x128(const uint16_t* x, int rows, int K,
                                uint8_t* out, float* scale, float* descale);

/* ---- elementwise epilogue ops ------------------------------------------- */
void orc_swiglu_forward(const uint16_t* gate, const uint16_t* up, uint16_t* out, int n);
void orc_bias_add_strided_bf16(uint16_t* inout, const uint16_t* bias,
                               int rows, int cols, int row_stride, int base);
/* swiglu_backward (kernels/activations.cu:42-58, 89-106) and the bias gradient col_sum_strided_bf16
 * (kernels/moe.cu:335-348, 357-364).  Pins: grad_up equals the forward applied to (gate, grad_out) bit for bit
 * (one commutative product), grad_gate against the closed form in double to half a bf16 ulp; the column sum
 * against numpy on exactly summable integers and on a column whose sequential sum differs from every tree. */
void orc_swiglu_backward(const uint16_t* grad_out, const uint16_t* gate, const uint16_t* up,
                         uint16_t* grad_gate, uint16_t* grad_up, int n);
void orc_col_sum_strided_bf16(const uint16_t* in, float* out_accum, int rows, int cols, int row_stride, int base);

/* ---- producers of the quantizer's input (cf_oracle_norm.c) ----------------
 * RMSNorm forward (kernels/rmsnorm.cu:13-54,101-108) and the absolute-ceiling
 * row clip (src/trainer.cu:3822-3842,3940-3991), both with the reference's
 * reduction trees.  orc_rmsnorm_forward returns non-zero when min(H,512) is
 * not a multiple of 32. */
int  orc_rmsnorm_forward(const uint16_t* x, const uint16_t* scale, uint16_t* out, float* rms,
                         int rows, int H, float eps);
void orc_act_row_clip_abs(uint16_t* x, int rows, int cols, float ceiling, float* normsq);

/* ---- chunked cross-entropy (cf_oracle_ce.c; kernels/cross_entropy.cu:201-305) ---- */
void orc_cross_entropy_count_valid(const int32_t* labels, int n, int* n_valid);
void orc_cross_entropy_fwd_bwd_chunk(const uint16_t* logits, const int32_t* labels, float* loss_out,
                                     uint16_t* grad, int rows, int V, const int* n_valid);

/* ---- MoE expert-bank backward helpers (cf_oracle_moe_bwd.c; kernels/moe.cu:510-521,623-674,1148-1167) ---- */
void orc_gelu_forward_bf16(const uint16_t* x, uint16_t* out, size_t n);
void orc_gelu_backward_bf16(const uint16_t* pre, const uint16_t* d_post, uint16_t* d_pre, size_t n);
void orc_moe_row_dot_selected_bf16(const uint16_t* a_full, const uint16_t* b_compact, float* out,
                                   const int* row_indices, int n_rows, int H, int out_stride, int out_col);
void orc_moe_gather_scale_rows_bf16(const uint16_t* src, uint16_t* dst, const float* route_weights,
                                    const int* row_indices, int n_rows, int expert_idx, int num_experts, int H);
void orc_moe_scatter_add_rows_bf16(uint16_t* dst_full, const uint16_t* src_compact, const int* row_indices,
                                   int n_rows, int H);

/* ---- GEMM references ----------------------------------------------------
 * scale_mode: 0 per-tensor (a_descale[1], b_descale[1])
 *             1 per-row / per-channel (a_descale[M], b_descale[N])
 *             2 block (a_descale[M, ceil(K/128)], b_descale[ceil(N/128), ceil(K/128)])
 * out_ref[M,N] (double accumulate of the fp32 dequantised operands) and
 * abs_dot[M,N] = sum_k |a_k*b_k| (the scale of an fp32 accumulation-order
 * difference); either may be NULL. */
void orc_gemm_nt_ref(int M, int N, int K,
                     const uint8_t* A, int lda, int a_is_e5m2, const float* a_descale,
                     const uint8_t* B, int ldb, int b_is_e5m2, const float* b_descale,
                     int scale_mode, double* out_ref, double* abs_dot, int threads);
/* Config-1 CPU path: Y[t,n] = bf16(dot_k(xq[t,k], wq[n,k])) with fp32
 * sequential accumulate over dequantised fp32 operands, rows split over
 * `threads` std::thread-style workers (src/cpu_trainer.cpp:89-108,306-324). */
void orc_linear_forward_f32(const float* xq, const float* wq, const uint16_t* bias,
                            uint16_t* y, int T, int K, int N, int threads);
void orc_dequant_n(const uint8_t* q, int is_e5m2, float descale, float* out, size_t n);

/* ---- MoE routing / dispatch (kernels/moe.cu, kernels/cross_entropy.cu) -- */
void orc_softmax_inplace_f32(float* x, int rows, int cols);
void orc_moe_topk_route_f32(float* scores, int rows, int num_experts, int top_k,
                            float* row_sum_save, float* scores_save, int normalize_topk);
void orc_moe_build_expert_row_lists(const float* route_weights, int* counts, int* row_indices,
                                    int rows, int num_experts);
void orc_moe_expert_offsets_from_counts(const int* counts, int* offsets, int num_experts);
void orc_moe_gather_rows_u8(const uint8_t* src, uint8_t* dst, const int* row_indices,
                            int n_rows, int width);
void orc_moe_gather_rows_bf16(const uint16_t* src, uint16_t* dst, const int* row_indices,
                              int n_rows, int width);
void orc_moe_scatter_accumulate_rows_bf16(uint16_t* mixed, const uint16_t* compact,
                                          const float* route_weights, const int* row_indices,
                                          int n_rows, int expert_idx, int num_experts, int H);
void orc_moe_scale_accumulate_bf16(uint16_t* mixed, const uint16_t* term,
                                   const float* route_weights, int rows, int expert_idx,
                                   int num_experts, int H);
/* Grouped GELU expert bank (kernels/moe.cu:950-1060): double-accumulated
 * reference of mixed[row] += w * fc_out(gelu(fc_in(hidden[row]))) for every
 * selected (expert,row) pair; mixed_ref is fp64 [rows,H] and must be preset to
 * the starting contents of mixed. */
void orc_moe_grouped_expert_forward_fp8_ref(
    const uint8_t* hidden, float fcin_descale, int fcin_is_e5m2,
    const float* route_weights, const int* counts, const int* row_indices,
    const uint8_t* fc_in_w, float fc_in_descale,
    const uint8_t* fc_out_w, float fc_out_descale,
    double* mixed_ref, int rows, int H, int Ie, int num_experts, int threads);

#ifdef __cplusplus
}
#endif
#endif
