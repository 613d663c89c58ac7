// The selected-expert backward of the GELU expert bank for every expert in one call.
//
// The reference walks the experts on the host (src/trainer.cu:7669-7741; the counts were copied to the host in the
// forward): per expert it recomputes the forward from the FP8 hidden states (gather, lt_gemm_fp8_nt fc_in,
// gelu_forward, quantize, lt_gemm_fp8_nt fc_out), takes the route-weight gradient as a row dot with d_mixed, scales
// d_mixed by the route weight into the expert's output gradient, and runs the four bf16 GEMMs, gelu_backward and the
// scatter-add of the input gradient: 16 launches per expert.  Here the same stages run once over the forward's saved
// counts / offsets / row_indices, experts back to back in compact buffers:
//
//   index   = the experts' row lists back to back                                     (moe_gather_rows_u8's order)
//   pre     = hidden_fp8[index] . fc_in_w8[e]^T              grouped FP8 GEMM, gather fused        src/trainer.cu:7688-7697
//   post    = gelu_forward(pre)                                                                     :7703
//   postq   = e4m3(post), one scale per token row            (the loop keeps a per-expert delayed scale: host-side state)
//   out     = postq . fc_out_w8[e]^T                          grouped FP8 GEMM                      :7713-7718
//   d_rw    = dot(d_mixed[row], out[slot]);  d_out = bf16(w . d_mixed[row])   over `out`           :7722-7725
//   g_out  += d_out^T . post                                  grouped bf16 GEMM (tn)                :7727
//   d_post  = d_out . fc_out_w[e]                             grouped bf16 GEMM (nn)                :7729
//   d_pre   = gelu_backward(pre, d_post)                                                            :7731
//   x       = hidden_bf16[index]                                                                    :7734
//   g_in   += d_pre^T . x                                     grouped bf16 GEMM (tn)                :7735
//   d_x     = d_pre . fc_in_w[e]                              grouped bf16 GEMM (nn)                :7737
//   d_hidden[row] += d_x[slot], experts in ascending order                                          :7739
//
// Nothing here is a kernel of its own except the clearing of the route-weight gradient: the stages are the library's
// entry points, enqueued on one stream with no host synchronisation.
#include "common.hpp"
#include "internal.hpp"

namespace cf {
namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void k_zero_f32(float* __restrict__ p, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        p[i] = 0.0f;
}
__global__ __launch_bounds__(kThreads) void k_zero_i32(int* __restrict__ p, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        p[i] = 0;
}
__global__ __launch_bounds__(kThreads) void k_spread3(const float* __restrict__ a, float* __restrict__ av, size_t na,
                                                      const float* __restrict__ b, float* __restrict__ bv, size_t nb,
                                                      const float* __restrict__ c, float* __restrict__ cv, size_t nc) {
    const float fa = *a, fb = *b, fc = *c;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < na + nb + nc;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        if (i < na) av[i] = fa;
        else if (i < na + nb) bv[i - na] = fb;
        else cv[i - na - nb] = fc;
    }
}

struct Layout { size_t off[CF_MOE_BWD_WS_COUNT]; size_t counts; size_t total; };

// counts[e] cut to what the compact buffers hold: total_rows is the caller's bound on the selected rows (the
// reference's callers pass rows * top_k), and every later stage walks (these counts, the caller's offsets)
__global__ __launch_bounds__(kThreads) void k_clamp_counts(const int* __restrict__ counts, const int* __restrict__ offsets, int E,
                                                           int total_rows, int* __restrict__ out) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const int first = offsets[e];
    out[e] = first >= 0 && first < total_rows ? max(0, min(counts[e], total_rows - first)) : 0;
}

Layout layout(int rows, int total_rows, int E, int H, int Ie) {
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t t = static_cast<size_t>(total_rows);
    size_t map_bytes = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_rows, E, &map_bytes);
    const size_t bytes[CF_MOE_BWD_WS_COUNT] = {
        /* CF_MOE_BWD_WS_TILE_MAP       */ map_bytes,
        /* CF_MOE_BWD_WS_INDEX          */ sizeof(int) * t,
        /* CF_MOE_BWD_WS_HIDDEN_DESCALE */ sizeof(float) * static_cast<size_t>(rows),
        /* CF_MOE_BWD_WS_IN_DESCALE     */ sizeof(float) * static_cast<size_t>(E) * Ie,
        /* CF_MOE_BWD_WS_OUT_DESCALE    */ sizeof(float) * static_cast<size_t>(E) * H,
        /* CF_MOE_BWD_WS_PRE            */ 2 * t * Ie,
        /* CF_MOE_BWD_WS_POST           */ 2 * t * Ie,
        /* CF_MOE_BWD_WS_POSTQ          */ t * Ie,
        /* CF_MOE_BWD_WS_POST_SCALE     */ sizeof(float) * t,
        /* CF_MOE_BWD_WS_POST_DESCALE   */ sizeof(float) * t,
        /* CF_MOE_BWD_WS_D_OUT          */ 2 * t * H,
        /* CF_MOE_BWD_WS_D_POST         */ 2 * t * Ie,
        /* CF_MOE_BWD_WS_D_PRE          */ 2 * t * Ie,
        /* CF_MOE_BWD_WS_X              */ 2 * t * H,
        /* CF_MOE_BWD_WS_D_X            */ 2 * t * H,
    };
    Layout l{};
    size_t at = 0;
    for (int i = 0; i < CF_MOE_BWD_WS_COUNT; ++i) {
        l.off[i] = at;
        at = up(at + bytes[i]);
    }
    l.counts = at;
    at = up(at + sizeof(int) * static_cast<size_t>(E));
    l.total = at;
    return l;
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_moe_grouped_gelu_backward_workspace(int rows, int total_selected_rows, int num_experts, int H, int Ie,
                                           size_t* offsets, size_t* bytes) {
    if (rows < 0 || total_selected_rows < 0 || num_experts < 0 || H < 0 || Ie < 0 || !bytes) return CF_ERR_INVALID_ARG;
    const Layout l = layout(rows, total_selected_rows, num_experts, H, Ie);
    if (offsets)
        for (int i = 0; i < CF_MOE_BWD_WS_COUNT; ++i) offsets[i] = l.off[i];
    *bytes = l.total;
    return CF_OK;
}

namespace {
struct FcoutSlots { float* states; int stride, history_len, is_e5m2; };

int gelu_bank_backward(const uint16_t* d_grad_mixed, const void* d_hidden_fp8, const float* d_fcin_descale,
                       int fcin_is_e5m2, const uint16_t* d_hidden_bf16, const float* d_route_weights,
                       const int* d_counts, const int* d_offsets, const int* d_row_indices,
                       const void* d_fc_in_w8, const float* d_fc_in_descale, const void* d_fc_out_w8,
                       const float* d_fc_out_descale, const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w,
                       float* d_grad_route_weights, uint16_t* d_grad_fc_in, uint16_t* d_grad_fc_out,
                       uint16_t* d_grad_hidden, int rows, int H, int Ie, int num_experts,
                       int total_selected_rows, const FcoutSlots& slots, void* d_workspace, size_t workspace_bytes, cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0 || total_selected_rows < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0) return CF_OK;
    if (!d_grad_mixed || !d_hidden_fp8 || !d_fcin_descale || !d_hidden_bf16 || !d_route_weights || !d_counts || !d_offsets ||
        !d_row_indices || !d_fc_in_w8 || !d_fc_in_descale || !d_fc_out_w8 || !d_fc_out_descale || !d_fc_in_w || !d_fc_out_w ||
        !d_grad_route_weights || !d_grad_fc_in || !d_grad_fc_out || !d_grad_hidden || !d_workspace)
        return CF_ERR_INVALID_ARG;
    const Layout l = layout(rows, total_selected_rows, num_experts, H, Ie);
    if (workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(d_workspace) & 255u)) return CF_ERR_INVALID_ARG;
    auto* base = static_cast<uint8_t*>(d_workspace);
    auto at = [&](int which) { return base + l.off[which]; };
    int* index = reinterpret_cast<int*>(at(CF_MOE_BWD_WS_INDEX));
    auto* hidden_descale = reinterpret_cast<float*>(at(CF_MOE_BWD_WS_HIDDEN_DESCALE));
    auto* in_descale = reinterpret_cast<float*>(at(CF_MOE_BWD_WS_IN_DESCALE));
    auto* out_descale = reinterpret_cast<float*>(at(CF_MOE_BWD_WS_OUT_DESCALE));
    auto* pre = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_PRE));
    auto* post = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_POST));
    auto* postq = at(CF_MOE_BWD_WS_POSTQ);
    auto* post_scale = reinterpret_cast<float*>(at(CF_MOE_BWD_WS_POST_SCALE));
    auto* post_descale = reinterpret_cast<float*>(at(CF_MOE_BWD_WS_POST_DESCALE));
    auto* d_out = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_D_OUT));
    auto* d_post = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_D_POST));
    auto* d_pre = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_D_PRE));
    auto* x = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_X));
    auto* d_x = reinterpret_cast<uint16_t*>(at(CF_MOE_BWD_WS_D_X));
    void* tile_map = at(CF_MOE_BWD_WS_TILE_MAP);
    size_t map_bytes = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_selected_rows, num_experts, &map_bytes);
    hipStream_t st = as_stream(stream);
    const int total = total_selected_rows;
    auto grid = [](size_t items) { return static_cast<unsigned>(min((items + kThreads - 1) / kThreads, static_cast<size_t>(2048))); };

    // the route-weight gradient starts from zero (cudaMemsetAsync at src/trainer.cu:7670-7672): cleared by a kernel, so
    // that the call can be recorded into a graph
    k_zero_f32<<<grid(static_cast<size_t>(rows) * num_experts), kThreads, 0, st>>>(d_grad_route_weights, static_cast<size_t>(rows) * num_experts);
    int rc = launch_status();
    if (rc) return rc;
    if (total == 0) return CF_OK;
    {
        const size_t na = static_cast<size_t>(rows), nb = static_cast<size_t>(num_experts) * Ie, nc = static_cast<size_t>(num_experts) * H;
        k_spread3<<<grid(na + nb + nc), kThreads, 0, st>>>(d_fcin_descale, hidden_descale, na, d_fc_in_descale, in_descale, nb,
                                                           d_fc_out_descale, out_descale, nc);
    }
    if ((rc = launch_status())) return rc;
    // total_selected_rows bounds the selected rows from above (the reference's callers pass rows * top_k,
    // src/trainer.cu:6863): no stage may go past it, whatever the counts say
    {
        int* clamped = reinterpret_cast<int*>(base + l.counts);
        k_clamp_counts<<<(num_experts + kThreads - 1) / kThreads, kThreads, 0, st>>>(d_counts, d_offsets, num_experts, total, clamped);
        if ((rc = launch_status())) return rc;
        d_counts = clamped;
    }
    // entries of the index past the experts' lists (a total above the sum of the counts) point at row 0: the
    // elementwise stages run over all `total` rows and must not gather from a stale index
    k_zero_i32<<<grid(static_cast<size_t>(total)), kThreads, 0, st>>>(index, static_cast<size_t>(total));
    if ((rc = launch_status())) return rc;
    if ((rc = cf_moe_compact_row_index(d_counts, d_offsets, d_row_indices, rows, num_experts, index, stream))) return rc;

    // ---- recompute of the forward from the FP8 hidden states ----
    if ((rc = grouped_gemm_nt_bf16(total, Ie, H, num_experts, d_counts, d_offsets, d_hidden_fp8, rows, H, index, hidden_descale,
                                   d_fc_in_w8, in_descale, CF_SCALE_ROW_COL, CF_EPI_NONE, nullptr, nullptr, pre, Ie, tile_map, map_bytes,
                                   true, fcin_is_e5m2 ? 1 : 0, stream)))
        return rc;
    if ((rc = cf_gelu_forward_bf16(pre, post, static_cast<size_t>(total) * Ie, stream))) return rc;
    // one scale per token row, or the recompute call of fp8_quant_act on the expert's slot (is_recompute = true: the
    // scale the forward's call snapshotted, no side effects; src/trainer.cu:7707-7712)
    if (slots.states)
        rc = cf_moe_grouped_quantize_delayed(post, postq, Ie, num_experts, d_counts, d_offsets, total, slots.states, slots.stride,
                                             slots.history_len, slots.is_e5m2, 0, 1, post_descale, stream);
    else
        rc = cf_fp8_quantize_rows(post, total, Ie, 0, postq, post_scale, post_descale, stream);
    if (rc) return rc;
    if ((rc = grouped_gemm_nt_bf16(total, H, Ie, num_experts, d_counts, d_offsets, postq, total, Ie, nullptr, post_descale,
                                   d_fc_out_w8, out_descale, CF_SCALE_ROW_COL, CF_EPI_NONE, nullptr, nullptr, d_out, H, tile_map, map_bytes,
                                   false, slots.states && slots.is_e5m2 ? 1 : 0, stream)))
        return rc;

    // ---- route-weight gradient; the expert outputs become their gradients in place ----
    if ((rc = cf_moe_grouped_route_grad_bf16(d_grad_mixed, d_out, d_grad_route_weights, d_route_weights, d_counts, d_offsets,
                                             d_row_indices, rows, num_experts, H, stream)))
        return rc;

    // ---- fc_out: weight gradient and input gradient ----
    if ((rc = cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, num_experts, d_counts, d_offsets, d_out, H, post, Ie, d_grad_fc_out, stream)))
        return rc;
    if ((rc = cf_moe_grouped_gemm_bf16_nn(total, Ie, H, num_experts, d_counts, d_offsets, d_out, H, d_fc_out_w, d_post, Ie, tile_map, map_bytes,
                                          stream)))
        return rc;
    if ((rc = cf_gelu_backward_bf16(pre, d_post, d_pre, static_cast<size_t>(total) * Ie, stream))) return rc;

    // ---- fc_in: weight gradient and input gradient ----
    if ((rc = cf_moe_gather_rows_bf16(d_hidden_bf16, x, index, total, H, stream))) return rc;
    if ((rc = cf_moe_grouped_gemm_bf16_tn_accum_bf16(Ie, H, total, num_experts, d_counts, d_offsets, d_pre, Ie, x, H, d_grad_fc_in, stream)))
        return rc;
    if ((rc = cf_moe_grouped_gemm_bf16_nn(total, H, Ie, num_experts, d_counts, d_offsets, d_pre, Ie, d_fc_in_w, d_x, H, tile_map, map_bytes,
                                          stream)))
        return rc;
    return cf_moe_unpermute_add_bf16(d_grad_hidden, d_x, d_route_weights, d_counts, d_offsets, d_row_indices, rows, num_experts, H,
                                     stream);
}
}  // namespace

int cf_moe_grouped_gelu_backward_fp8(const uint16_t* d_grad_mixed, const void* d_hidden_fp8, const float* d_fcin_descale,
                                     int fcin_is_e5m2, const uint16_t* d_hidden_bf16, const float* d_route_weights,
                                     const int* d_counts, const int* d_offsets, const int* d_row_indices,
                                     const void* d_fc_in_w8, const float* d_fc_in_descale, const void* d_fc_out_w8,
                                     const float* d_fc_out_descale, const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w,
                                     float* d_grad_route_weights, uint16_t* d_grad_fc_in, uint16_t* d_grad_fc_out,
                                     uint16_t* d_grad_hidden, int rows, int H, int Ie, int num_experts,
                                     int total_selected_rows, void* d_workspace, size_t workspace_bytes, cf_stream_t stream) {
    return gelu_bank_backward(d_grad_mixed, d_hidden_fp8, d_fcin_descale, fcin_is_e5m2, d_hidden_bf16, d_route_weights, d_counts, d_offsets,
                              d_row_indices, d_fc_in_w8, d_fc_in_descale, d_fc_out_w8, d_fc_out_descale, d_fc_in_w, d_fc_out_w,
                              d_grad_route_weights, d_grad_fc_in, d_grad_fc_out, d_grad_hidden, rows, H, Ie, num_experts,
                              total_selected_rows, FcoutSlots{nullptr, 0, 0, 0}, d_workspace, workspace_bytes, stream);
}

int cf_moe_grouped_gelu_backward_fp8_slots(const uint16_t* d_grad_mixed, const void* d_hidden_fp8, const float* d_fcin_descale,
                                           int fcin_is_e5m2, const uint16_t* d_hidden_bf16, const float* d_route_weights,
                                           const int* d_counts, const int* d_offsets, const int* d_row_indices,
                                           const void* d_fc_in_w8, const float* d_fc_in_descale, const void* d_fc_out_w8,
                                           const float* d_fc_out_descale, const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w,
                                           float* d_grad_route_weights, uint16_t* d_grad_fc_in, uint16_t* d_grad_fc_out,
                                           uint16_t* d_grad_hidden, int rows, int H, int Ie, int num_experts,
                                           int total_selected_rows, float* d_fcout_slot_states, int state_stride_words,
                                           int history_len, int fcout_is_e5m2, void* d_workspace, size_t workspace_bytes,
                                           cf_stream_t stream) {
    if (!d_fcout_slot_states || history_len < 0 || state_stride_words < cf_act_slot_state_words(history_len)) return CF_ERR_INVALID_ARG;
    return gelu_bank_backward(d_grad_mixed, d_hidden_fp8, d_fcin_descale, fcin_is_e5m2, d_hidden_bf16, d_route_weights, d_counts, d_offsets,
                              d_row_indices, d_fc_in_w8, d_fc_in_descale, d_fc_out_w8, d_fc_out_descale, d_fc_in_w, d_fc_out_w,
                              d_grad_route_weights, d_grad_fc_in, d_grad_fc_out, d_grad_hidden, rows, H, Ie, num_experts,
                              total_selected_rows, FcoutSlots{d_fcout_slot_states, state_stride_words, history_len, fcout_is_e5m2 ? 1 : 0},
                              d_workspace, workspace_bytes, stream);
}

}  // extern "C"
