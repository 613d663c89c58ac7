// Host-side FP8 slot state machines: the per-call-site delayed-scaling activation slot
// (calibration, first use, steady state, recompute) and the per-weight refresh, expressed
// over the quantize entry points of this library.  Device scalars live in one caller-owned
// block; the host object only carries the flags the reference keeps in its slot struct.
#include "common.hpp"
#include "internal.hpp"

#include <new>

struct cf_act_slot {
    float* state;              // device block, layout below
    int history_len;
    float fp8_max;
    bool init;
    int calib_remaining;
    bool calib_commit_pending;
    float spread_threshold;
};

namespace cf {
namespace {

// device block layout, in 4-byte words
enum { W_AMAX = slotw::AMAX, W_SCALE = slotw::SCALE, W_DESCALE = slotw::DESCALE, W_SCALE_SNAP = slotw::SCALE_SNAP,
       W_DESCALE_SNAP = slotw::DESCALE_SNAP, W_CALIB_MIN = slotw::CALIB_MIN, W_CALIB_MAX = slotw::CALIB_MAX, W_CURSOR = slotw::CURSOR,
       W_COUNT = slotw::COUNT, W_RUNNING_AMAX = slotw::RUNNING, W_ARRIVED = slotw::ARRIVED, W_HISTORY = slotw::HISTORY };

__global__ void k_slot_init(float* st, int history_len) {
    for (int i = threadIdx.x; i < W_HISTORY + history_len; i += blockDim.x) st[i] = 0.0f;   // zero words are int 0 as well
    __syncthreads();
    if (threadIdx.x == 0) st[W_CALIB_MIN] = __uint_as_float(0x7f7f7f7fu);                    // "min so far" sentinel, ~3.39e38
}
__global__ void k_snapshot(float* st) {
    st[W_SCALE_SNAP] = st[W_SCALE];
    st[W_DESCALE_SNAP] = st[W_DESCALE];
}
__global__ void k_zero_amax(float* st) { st[W_AMAX] = 0.0f; }
__global__ void k_commit_e5m2(float* st) {
    st[W_AMAX] = st[W_CALIB_MAX];
    reinterpret_cast<int*>(st)[W_CURSOR] = 0;
    reinterpret_cast<int*>(st)[W_COUNT] = 0;
}

int quantize(const cf_act_slot* s, const uint16_t* x, void* out, const float* scale, float* amax_record, size_t n, cf_stream_t st) {
    const bool e5m2 = s->fp8_max == CF_E5M2_MAX;
    if (amax_record)
        return e5m2 ? cf_fp8_quantize_e5m2_record(x, out, scale, amax_record, n, st) : cf_fp8_quantize_e4m3_record(x, out, scale, amax_record, n, st);
    return e5m2 ? cf_fp8_quantize_e5m2(x, out, scale, n, st) : cf_fp8_quantize_e4m3(x, out, scale, n, st);
}

int update_history(cf_act_slot* s, cf_stream_t st) {
    float* d = s->state;
    return cf_fp8_update_delayed_scale(d + W_AMAX, s->fp8_max, d + W_SCALE, d + W_DESCALE, d + W_HISTORY, s->history_len,
                                       reinterpret_cast<int*>(d) + W_CURSOR, reinterpret_cast<int*>(d) + W_COUNT, st);
}

}  // namespace
}  // namespace cf

using namespace cf;

#define CF_TRY(expr) do { const int rc_ = (expr); if (rc_ != CF_OK) return rc_; } while (0)

extern "C" {

int cf_act_slot_state_words(int history_len) { return W_HISTORY + (history_len > 0 ? history_len : 0); }

int cf_act_slot_create(cf_act_slot** out, void* d_state, int history_len, float fp8_max, int calib_calls,
                       float type_spread_threshold, cf_stream_t stream) {
    if (!out || !d_state || history_len < 0 || calib_calls < 0) return CF_ERR_INVALID_ARG;
    if (fp8_max != CF_E4M3_MAX && fp8_max != CF_E5M2_MAX) return CF_ERR_INVALID_ARG;
    cf_act_slot* s = new (std::nothrow) cf_act_slot{};
    if (!s) return CF_ERR_INVALID_ARG;
    s->state = static_cast<float*>(d_state);
    s->history_len = history_len;
    s->fp8_max = fp8_max;
    s->init = false;
    s->calib_remaining = calib_calls;
    s->calib_commit_pending = false;
    s->spread_threshold = type_spread_threshold > 1.0f ? type_spread_threshold : 4.0f;
    k_slot_init<<<1, 64, 0, as_stream(stream)>>>(s->state, history_len);
    const int rc = launch_status();
    if (rc != CF_OK) { delete s; return rc; }
    *out = s;
    return CF_OK;
}

int cf_act_slot_destroy(cf_act_slot* slot) {
    delete slot;
    return CF_OK;
}

int cf_act_slot_is_e5m2(const cf_act_slot* slot) { return slot && slot->fp8_max == CF_E5M2_MAX; }

int cf_act_slot_device_field(const cf_act_slot* slot, int field, void** d_ptr) {
    if (!slot || !d_ptr) return CF_ERR_INVALID_ARG;
    static const int word[] = {W_AMAX, W_SCALE, W_DESCALE, W_SCALE_SNAP, W_DESCALE_SNAP, W_HISTORY, W_CURSOR, W_COUNT, W_CALIB_MIN, W_CALIB_MAX};
    if (field < 0 || field >= static_cast<int>(sizeof(word) / sizeof(word[0]))) return CF_ERR_INVALID_ARG;
    *d_ptr = slot->state + word[field];
    return CF_OK;
}

int cf_fp8_quant_act(cf_act_slot* slot, const uint16_t* d_x, void* d_act8, size_t n, int is_recompute, cf_stream_t stream) {
    if (!slot || (n > 0 && (!d_x || !d_act8))) return CF_ERR_INVALID_ARG;
    float* d = slot->state;
    hipStream_t st = as_stream(stream);
    if (is_recompute)      // same scale the forward call used, no side effects
        return quantize(slot, d_x, d_act8, d + W_SCALE_SNAP, nullptr, n, stream);

    // a pending calibration decision is committed before this call quantizes, never between a forward and its recompute
    if (slot->calib_commit_pending) {
        slot->calib_commit_pending = false;
        float mn = 0.0f, mx = 0.0f;
        hipError_t e = hipStreamSynchronize(st);
        if (e == hipSuccess) e = hipMemcpy(&mn, d + W_CALIB_MIN, sizeof(float), hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(&mx, d + W_CALIB_MAX, sizeof(float), hipMemcpyDeviceToHost);
        if (e != hipSuccess) return static_cast<int>(e);
        const float spread = mn > 0.0f ? mx / mn : 0.0f;
        if (slot->fp8_max == CF_E4M3_MAX && spread > slot->spread_threshold) {
            // the range moves too much for E4M3: commit to E5M2 and reseed the delayed state from the widest amax seen
            slot->fp8_max = CF_E5M2_MAX;
            k_commit_e5m2<<<1, 1, 0, st>>>(d);
            CF_TRY(launch_status());
            CF_TRY(cf_fp8_scale_from_amax(d + W_AMAX, slot->fp8_max, d + W_SCALE, d + W_DESCALE, stream));
            CF_TRY(update_history(slot, stream));
        }
    }

    if (slot->calib_remaining > 0 || !slot->init) {
        k_zero_amax<<<1, 1, 0, st>>>(d);
        CF_TRY(launch_status());
        // exact per-call amax (no stale scale); during calibration the spread of the amax is recorded too
        CF_TRY(cf_fp8_amax_bf16(d_x, n, d + W_AMAX, stream));
        CF_TRY(cf_fp8_scale_from_amax(d + W_AMAX, slot->fp8_max, d + W_SCALE, d + W_DESCALE, stream));
        k_snapshot<<<1, 1, 0, st>>>(d);
        CF_TRY(launch_status());
        CF_TRY(quantize(slot, d_x, d_act8, d + W_SCALE, nullptr, n, stream));
        if (slot->calib_remaining > 0) CF_TRY(cf_fp8_calib_minmax_update(d + W_AMAX, d + W_CALIB_MIN, d + W_CALIB_MAX, stream));
        CF_TRY(update_history(slot, stream));
        slot->init = true;
        if (slot->calib_remaining > 0 && --slot->calib_remaining == 0) slot->calib_commit_pending = true;
        return CF_OK;
    }
    // steady state: snapshot the pair the GEMM will dequantize with, quantize with the PREVIOUS scale while recording
    // this tensor's amax, then advance the history -- one launch
    return cf_fp8_quantize_delayed_step(d_x, d_act8, n, slot->fp8_max == CF_E5M2_MAX, d + W_AMAX, d + W_SCALE, d + W_DESCALE,
                                        d + W_SCALE_SNAP, d + W_DESCALE_SNAP, d + W_HISTORY, slot->history_len,
                                        reinterpret_cast<int*>(d) + W_CURSOR, reinterpret_cast<int*>(d) + W_COUNT,
                                        d + W_RUNNING_AMAX, reinterpret_cast<unsigned int*>(d) + W_ARRIVED, stream);
}

int cf_fp8_refresh_weight(const uint16_t* d_w, void* d_fwd8, void* d_bwd8, float* d_amax, float* d_scale, float* d_descale,
                          int in_dim, int out_dim, int stored_out_major, int recompute_amax, cf_stream_t stream) {
    if (in_dim < 0 || out_dim < 0) return CF_ERR_INVALID_ARG;
    if (!d_w || !d_fwd8 || !d_bwd8 || !d_amax || !d_scale || !d_descale) return CF_ERR_INVALID_ARG;
    const size_t n = static_cast<size_t>(in_dim) * out_dim;
    if (recompute_amax) CF_TRY(cf_fp8_amax_bf16(d_w, n, d_amax, stream));
    CF_TRY(cf_fp8_scale_from_amax(d_amax, CF_E4M3_MAX, d_scale, d_descale, stream));
    // Both layouts from one read of the weight (the dual quantize gives the same bytes as the reference's two
    // kernels, fp8_quantize_e4m3 and fp8_quantize_transpose_e4m3: same scale, same conversion).
    if (stored_out_major)   // stored [out,in]: the direct quantize is the forward layout, the transposed one the backward layout
        return cf_fp8_quant_and_transpose_e4m3(d_w, d_fwd8, d_bwd8, d_scale, out_dim, in_dim, stream);
    return cf_fp8_quant_and_transpose_e4m3(d_w, d_bwd8, d_fwd8, d_scale, in_dim, out_dim, stream);
}

}  // extern "C"
