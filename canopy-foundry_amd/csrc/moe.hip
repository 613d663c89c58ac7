// MoE routing and dispatch for gfx950: row softmax, top-k select + renormalise,
// deterministic per-expert row lists, offsets, row gather (token permute) and the
// weighted scatter-accumulate (unpermute).
//
// Routing is bit-reproducible: the softmax uses the library's deterministic expf and
// a fixed reduction tree (32-lane xor butterflies, then the group sums), top-k picks
// by (value descending, index ascending), and row lists are filled in ascending row
// order by a scan instead of atomics.
#include "common.hpp"
#include "internal.hpp"

#include <mutex>
#include <type_traits>

namespace cf {
namespace {

constexpr int kThreads = 256;

// xor butterfly over the 32-lane group a lane belongs to (offsets 16..1)
__device__ __forceinline__ float group32_sum(float v) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float group32_max(float v) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// ---- softmax, cols <= 64: one wavefront per row, lane = column ----------------
// Matches a launch of T = cols threads: one element per thread, 32-lane butterflies,
// then the (at most two) group sums added.
__device__ __forceinline__ float row_softmax_wave(float x, bool live, float& out_max) {
    const float m32 = group32_max(live ? x : -3.402823466e+38f);
    const float mx = fmaxf(m32, __shfl_xor(m32, 32, kWave));
    const float e = live ? det_expf(x - mx) : 0.0f;
    const float s32 = group32_sum(e);
    // second level: the butterfly over {s_lo, s_hi, 0, ...} reduces to s_lo + s_hi
    const float lo = __shfl(s32, 0, kWave), hi = __shfl(s32, 32, kWave);
    const float sum = lo + hi;
    const float inv = 1.0f / sum;
    out_max = mx;
    return e * inv;
}

__global__ __launch_bounds__(kThreads) void k_softmax_wave(float* __restrict__ x, int rows, int cols) {
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const bool live = lane < cols;
    float* r = x + static_cast<size_t>(row) * cols;
    float mx;
    const float p = row_softmax_wave(live ? r[lane] : 0.0f, live, mx);
    if (live) r[lane] = p;
}

// ---- softmax, any cols: one workgroup per row, T = min(cols,256) virtual threads ----
__global__ __launch_bounds__(kThreads) void k_softmax_block(float* __restrict__ x, int cols) {
    __shared__ float sh[8];
    __shared__ float bc;
    float* r = x + static_cast<size_t>(blockIdx.x) * cols;
    const int T = min(cols, 256), t = threadIdx.x;
    float lm = -3.402823466e+38f;
    if (t < T) for (int c = t; c < cols; c += T) lm = fmaxf(lm, r[c]);
    lm = group32_max(lm);
    if ((t & 31) == 0) sh[t >> 5] = lm;
    __syncthreads();
    if (t == 0) { float m = sh[0]; for (int w = 1; w < 8; ++w) m = fmaxf(m, sh[w]); bc = m; }
    __syncthreads();
    const float mx = bc;
    float ls = 0.0f;
    if (t < T) for (int c = t; c < cols; c += T) ls += det_expf(r[c] - mx);
    ls = group32_sum(ls);
    __syncthreads();
    if ((t & 31) == 0) sh[t >> 5] = ls;          // groups past T hold 0
    __syncthreads();
    if (t == 0) {
        // butterfly over the 32-entry array of group sums (only the first 8 can be non-zero):
        // offsets 16 and 8 add zeros, then (w0+w4),(w1+w5),(w2+w6),(w3+w7); (.. + ..) pairs 2 apart; then 1 apart
        const float a0 = sh[0] + sh[4], a1 = sh[1] + sh[5], a2 = sh[2] + sh[6], a3 = sh[3] + sh[7];
        bc = (a0 + a2) + (a1 + a3);
    }
    __syncthreads();
    const float inv = 1.0f / bc;
    if (t < T) for (int c = t; c < cols; c += T) r[c] = det_expf(r[c] - mx) * inv;
}

// ---- top-k, E <= 64: one wavefront per row, lane = expert ----------------------
// Optionally fused with the softmax (SOFTMAX) so the logits are read once.
template <bool SOFTMAX>
__global__ __launch_bounds__(kThreads) void k_topk_wave(float* __restrict__ scores, float* __restrict__ row_sum_save,
                                                        float* __restrict__ scores_save, int rows, int E, int top_k,
                                                        int normalize) {
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const bool live = lane < E;
    float* s = scores + static_cast<size_t>(row) * E;
    float v = live ? s[lane] : 0.0f;
    if constexpr (SOFTMAX) {
        float mx;
        v = row_softmax_wave(v, live, mx);
        if (scores_save && live) scores_save[static_cast<size_t>(row) * E + lane] = v;
    }
    const int k = min(top_k, E);
    bool kept = false;
    for (int pick = 0; pick < k; ++pick) {
        // candidates must beat -1 strictly (NaN never does); largest value, lowest lane among equals
        const bool cand = live && !kept && v > -1.0f;
        float best = cand ? v : -2.0f;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) best = fmaxf(best, __shfl_xor(best, off, kWave));
        const unsigned long long hit = __ballot(cand && v == best);
        if (hit == 0ull) break;
        if (lane == __builtin_ctzll(hit)) kept = true;
    }
    // kept sum in ascending expert order, one fp32 add per kept expert
    unsigned long long mask = __ballot(kept);
    float sum = 0.0f;
    while (mask) {
        const int e = __builtin_ctzll(mask);
        mask &= mask - 1;
        sum += __shfl(v, e, kWave);
    }
    if (row_sum_save && lane == 0) row_sum_save[row] = sum;
    const float inv_sum = (normalize && sum > 0.0f) ? (1.0f / sum) : 1.0f;
    if (live) s[lane] = kept ? v * inv_sum : 0.0f;
}

// ---- top-k, 64 < E <= 2048: one wavefront per row, lane l holds experts l, l + 64, ... ----------
// A pick is the largest remaining score, the lowest expert among equals; scores must beat -1 strictly (NaN never
// does).  Each lane scans its own experts in ascending order, the wavefront agrees on the largest value and then on
// the lowest expert that holds it.  The kept sum runs in ascending expert order, one fp32 add per kept expert.
constexpr int kMaxExpertsGeneric = 2048;
__global__ __launch_bounds__(kThreads) void k_topk_wide(float* __restrict__ scores, float* __restrict__ row_sum_save,
                                                        int rows, int E, int top_k, int normalize) {
    constexpr int J = kMaxExpertsGeneric / 64;
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    float* s = scores + static_cast<size_t>(row) * E;
    float v[J];
#pragma unroll
    for (int j = 0; j < J; ++j) v[j] = j * 64 + lane < E ? s[j * 64 + lane] : -2.0f;
    uint32_t kept = 0u;            // bit j: expert j * 64 + lane is kept
    const int k = min(top_k, E);
    for (int pick = 0; pick < k; ++pick) {
        float best = -1.0f;
        int bj = -1;
#pragma unroll
        for (int j = 0; j < J; ++j)
            if (!((kept >> j) & 1u) && v[j] > best) { best = v[j]; bj = j; }
        float top = best;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, kWave));
        int who = (bj >= 0 && best == top) ? bj * 64 + lane : 0x7fffffff;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) who = min(who, __shfl_xor(who, off, kWave));
        if (who == 0x7fffffff) break;                      // nothing left that beats -1
        if ((who & 63) == lane) kept |= 1u << (who >> 6);
    }
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        unsigned long long mask = j * 64 < E ? __ballot((kept >> j) & 1u) : 0ull;
        while (mask) {
            const int l = __builtin_ctzll(mask);
            mask &= mask - 1;
            sum += __shfl(v[j], l, kWave);
        }
    }
    if (row_sum_save && lane == 0) row_sum_save[row] = sum;
    const float inv_sum = (normalize && sum > 0.0f) ? (1.0f / sum) : 1.0f;
#pragma unroll
    for (int j = 0; j < J; ++j)
        if (j * 64 + lane < E) s[j * 64 + lane] = ((kept >> j) & 1u) ? v[j] * inv_sum : 0.0f;
}

// ---- per-expert row lists ----------------------------------------------------------
// One workgroup per expert scans the rows 1024 at a time: ballot + popcount inside a
// wavefront, wavefront totals through LDS, so slots come out in ascending row order.
__global__ __launch_bounds__(1024) void k_build_row_lists(const float* __restrict__ route_weights,
                                                          int* __restrict__ counts, int* __restrict__ row_indices,
                                                          int rows, int E) {
    // One workgroup per expert walks its (strided) column in super-slabs of 16 x 1024 rows: all sixteen membership
    // loads of a lane are issued together (each is a full memory latency), the 256 per-(slab, wavefront) member
    // counts are scanned once, and every lane then writes its members at their ranks: ascending row order.
    __shared__ int tot[256];          // [slab][wavefront] member counts, then their exclusive prefix
    __shared__ int wsum[4];
    __shared__ int base_sh;
    const int e = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
    int* out = row_indices + static_cast<size_t>(e) * rows;
    if (t == 0) base_sh = 0;
    for (int r0 = 0; r0 < rows; r0 += 16 * 1024) {
        unsigned bits = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = r0 + i * 1024 + t;
            const float w = row < rows ? route_weights[static_cast<size_t>(row) * E + e] : 0.0f;
            bits |= (w > 0.0f ? 1u : 0u) << i;
        }
        int rank[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const unsigned long long m = __ballot((bits >> i) & 1u);
            rank[i] = __builtin_popcountll(m & ((1ull << lane) - 1ull));
            if (lane == 0) tot[i * 16 + wave] = __builtin_popcountll(m);
        }
        __syncthreads();
        // exclusive prefix of the 256 counts in (slab, wavefront) order by the first four wavefronts
        int incl = 0, mine = 0;
        if (t < 256) {
            mine = tot[t];
            incl = mine;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int o = __shfl_up(incl, off, kWave);
                if (lane >= off) incl += o;
            }
            if (lane == 63) wsum[wave] = incl;
        }
        __syncthreads();
        const int base = base_sh;
        if (t < 256) {
            int before = 0;
            for (int w = 0; w < wave; ++w) before += wsum[w];
            tot[t] = before + incl - mine;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 16; ++i)
            if ((bits >> i) & 1u) out[base + tot[i * 16 + wave] + rank[i]] = r0 + i * 1024 + t;
        __syncthreads();                                  // tot and base_sh are rewritten next
        if (t == 0) base_sh = base + wsum[0] + wsum[1] + wsum[2] + wsum[3];
        __syncthreads();
    }
    if (t == 0) counts[e] = base_sh;
}

__global__ void k_offsets(const int* __restrict__ counts, int* __restrict__ offsets, int E) {
    int sum = 0;
    for (int e = 0; e < E; ++e) { offsets[e] = sum; sum += counts[e]; }
}

// ---- row gather (token permute) -----------------------------------------------------
// dst[i, :] = src[row_indices[i], :], rows of `width` bytes; 16 bytes per lane when aligned.
__global__ __launch_bounds__(kThreads) void k_gather_rows16(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                            const int* __restrict__ row_indices, int n_rows,
                                                            int vec_per_row) {
    const size_t total = static_cast<size_t>(n_rows) * vec_per_row;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const int r = static_cast<int>(i / vec_per_row), c = static_cast<int>(i % vec_per_row);
        store_stream16(dst + i, src[static_cast<size_t>(row_indices[r]) * vec_per_row + c]);
    }
}
template <typename T>
__global__ __launch_bounds__(kThreads) void k_gather_rows_scalar(const T* __restrict__ src, T* __restrict__ dst,
                                                                 const int* __restrict__ row_indices, int n_rows,
                                                                 int width) {
    const size_t total = static_cast<size_t>(n_rows) * width;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const int r = static_cast<int>(i / width), c = static_cast<int>(i % width);
        dst[i] = src[static_cast<size_t>(row_indices[r]) * width + c];
    }
}

// ---- weighted scatter-accumulate (unpermute) -------------------------------------------
// mixed[row,h] = bf16(fma(w, compact[i,h], mixed[row,h])): one fused multiply-add (what the
// CUDA compiler makes of `m + w * c` by default) and one bf16 rounding.
__device__ __forceinline__ uint32_t fma2_bf16(uint32_t m, uint32_t c, float w) {
    const float lo = __builtin_fmaf(w, bf16_lo(c), bf16_lo(m));
    const float hi = __builtin_fmaf(w, bf16_hi(c), bf16_hi(m));
    return pack_bf16x2(lo, hi);
}
// rows of `compact` map to rows of `mixed` through row_indices (or identically when it is null); without route
// weights the factor is 1 and the operation is the plain add of the backward's scatter (fma(1, c, m) = m + c)
__global__ __launch_bounds__(kThreads) void k_scatter_accumulate(uint16_t* __restrict__ mixed,
                                                                 const uint16_t* __restrict__ compact,
                                                                 const float* __restrict__ route_weights,
                                                                 const int* __restrict__ row_indices, int n_rows,
                                                                 int expert_idx, int E, int H, int vec) {
    if (vec) {
        const int vpr = H / 8;
        const size_t total = static_cast<size_t>(n_rows) * vpr;
        for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
             i += static_cast<size_t>(gridDim.x) * blockDim.x) {
            const int r = static_cast<int>(i / vpr), c = static_cast<int>(i % vpr);
            const int row = row_indices ? row_indices[r] : r;
            const float w = route_weights ? route_weights[static_cast<size_t>(row) * E + expert_idx] : 1.0f;
            uint4* dst = reinterpret_cast<uint4*>(mixed + static_cast<size_t>(row) * H) + c;
            const uint4 cv = reinterpret_cast<const uint4*>(compact + static_cast<size_t>(r) * H)[c];
            uint4 mv = *dst;
            mv.x = fma2_bf16(mv.x, cv.x, w); mv.y = fma2_bf16(mv.y, cv.y, w);
            mv.z = fma2_bf16(mv.z, cv.z, w); mv.w = fma2_bf16(mv.w, cv.w, w);
            *dst = mv;
        }
    } else {
        const size_t total = static_cast<size_t>(n_rows) * H;
        for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
             i += static_cast<size_t>(gridDim.x) * blockDim.x) {
            const int r = static_cast<int>(i / H), h = static_cast<int>(i % H);
            const int row = row_indices ? row_indices[r] : r;
            const float w = route_weights ? route_weights[static_cast<size_t>(row) * E + expert_idx] : 1.0f;
            uint16_t* dst = mixed + static_cast<size_t>(row) * H + h;
            *dst = f32_to_bf16(__builtin_fmaf(w, bf16_to_f32(compact[i]), bf16_to_f32(*dst)));
        }
    }
}

// ---- compact row index: the row lists of all experts back to back --------------------
__global__ __launch_bounds__(kThreads) void k_compact_index(const int* __restrict__ counts, const int* __restrict__ offsets,
                                                            const int* __restrict__ row_indices, int rows,
                                                            int* __restrict__ compact, int* __restrict__ slot_index, int E) {
    const int e = blockIdx.y;
    const int n = counts[e], base = offsets[e];
    for (int s = blockIdx.x * blockDim.x + threadIdx.x; s < n; s += gridDim.x * blockDim.x) {
        const int row = row_indices[static_cast<size_t>(e) * rows + s];
        compact[base + s] = row;
        if (slot_index) slot_index[static_cast<size_t>(row) * E + e] = base + s;      // the inverse, for the unpermute
    }
}

// ---- fused weighted unpermute ------------------------------------------------------------
// One workgroup per token row.  For every expert with a positive route weight, in ascending expert
// order: mixed[row] = bf16(fma(w, y[slot], mixed[row])), slot = offsets[e] + rank of the row in the
// expert's (ascending) row list.  Same arithmetic and order as one scatter-accumulate launch per expert.
// The rank is found by a 64-ary search, one wavefront per selected expert: each round is one coalesced
// probe of 64 list entries, so a list of 4096 rows costs two memory latencies instead of twelve.

// Position of `row` in the ascending list[0, cnt), or -1.  Called by a whole wavefront.
__device__ __forceinline__ int wave_find_sorted(const int* __restrict__ list, int cnt, int row, int lane) {
    int lo = 0, len = cnt;
    while (len > 64) {
        const int stride = (len + 63) >> 6;
        const int idx = lo + lane * stride;
        const int v = idx < lo + len ? list[idx] : 0x7fffffff;
        const unsigned long long le = __ballot(v <= row);       // a prefix of the lanes: the list ascends
        if (le == 0) return -1;
        const int j = 63 - __builtin_clzll(le);
        const int end = lo + len;
        lo += j * stride;
        len = min(stride, end - lo);
    }
    const int v = lane < len ? list[lo + lane] : 0x7fffffff;
    const unsigned long long eq = __ballot(v == row);
    return eq ? lo + __builtin_ctzll(eq) : -1;
}

// mixed row += the n listed rows of y, in list order, one bf16 rounding per row (slot < 0: skipped)
__device__ __forceinline__ void combine_rows(uint16_t* __restrict__ mrow, const uint16_t* __restrict__ y, int H, int n,
                                             const int* sl_slot, const float* sl_w, int t) {
    if ((H & 7) == 0) {
        for (int c = t; c < H / 8; c += blockDim.x) {
            uint4 mv = reinterpret_cast<uint4*>(mrow)[c];
            for (int i0 = 0; i0 < n; i0 += 4) {
                // up to four rows of y in flight at once, applied in order
                uint4 yv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int slot = i0 + j < n ? sl_slot[i0 + j] : -1;
                    yv[j] = make_uint4(0, 0, 0, 0);
                    if (slot >= 0) yv[j] = reinterpret_cast<const uint4*>(y + static_cast<size_t>(slot) * H)[c];
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (i0 + j < n && sl_slot[i0 + j] >= 0) {
                        const float w = sl_w[i0 + j];
                        mv.x = fma2_bf16(mv.x, yv[j].x, w); mv.y = fma2_bf16(mv.y, yv[j].y, w);
                        mv.z = fma2_bf16(mv.z, yv[j].z, w); mv.w = fma2_bf16(mv.w, yv[j].w, w);
                    }
                }
            }
            store_stream16(reinterpret_cast<uint4*>(mrow) + c, mv);
        }
    } else {
        for (int h = t; h < H; h += blockDim.x) {
            float m = bf16_to_f32(mrow[h]);
            for (int i = 0; i < n; ++i)
                if (sl_slot[i] >= 0)
                    m = bf16_to_f32(f32_to_bf16(__builtin_fmaf(sl_w[i], bf16_to_f32(y[static_cast<size_t>(sl_slot[i]) * H + h]), m)));
            mrow[h] = f32_to_bf16(m);
        }
    }
}

// The same for fp32 rows of y: mixed = bf16(mixed + w * y) per listed row, product and sum rounded in fp32 as
// separate operations (what an add of the argument `w * y` to the stored value does), one bf16 rounding per row.
__device__ __forceinline__ uint32_t add2_bf16(uint32_t m, float y0, float y1, float w) {
    return pack_bf16x2(bf16_lo(m) + w * y0, bf16_hi(m) + w * y1);
}
__device__ __forceinline__ void combine_rows(uint16_t* __restrict__ mrow, const float* __restrict__ y, int H, int n,
                                             const int* sl_slot, const float* sl_w, int t) {
    if ((H & 7) == 0) {
        for (int c = t; c < H / 8; c += blockDim.x) {
            uint4 mv = reinterpret_cast<uint4*>(mrow)[c];
            for (int i0 = 0; i0 < n; i0 += 4) {
                float4 ya[4], yb[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int slot = i0 + j < n ? sl_slot[i0 + j] : -1;
                    ya[j] = yb[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    if (slot >= 0) {
                        const float4* src = reinterpret_cast<const float4*>(y + static_cast<size_t>(slot) * H) + 2 * c;
                        ya[j] = src[0]; yb[j] = src[1];
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (i0 + j < n && sl_slot[i0 + j] >= 0) {
                        const float w = sl_w[i0 + j];
                        mv.x = add2_bf16(mv.x, ya[j].x, ya[j].y, w); mv.y = add2_bf16(mv.y, ya[j].z, ya[j].w, w);
                        mv.z = add2_bf16(mv.z, yb[j].x, yb[j].y, w); mv.w = add2_bf16(mv.w, yb[j].z, yb[j].w, w);
                    }
                }
            }
            store_stream16(reinterpret_cast<uint4*>(mrow) + c, mv);
        }
    } else {
        for (int h = t; h < H; h += blockDim.x) {
            float m = bf16_to_f32(mrow[h]);
            for (int i = 0; i < n; ++i)
                if (sl_slot[i] >= 0) m = bf16_to_f32(f32_to_bf16(m + sl_w[i] * y[static_cast<size_t>(sl_slot[i]) * H + h]));
            mrow[h] = f32_to_bf16(m);
        }
    }
}

// The same with the slots read from a table slot_index[row, e] (filled by k_slot_index for the selected pairs):
// no search, so a row's critical path is one load of its weights and slots, then the gathers.
template <bool UNIT, class YT = uint16_t>
__global__ __launch_bounds__(kThreads) void k_unpermute_indexed(uint16_t* __restrict__ mixed, const YT* __restrict__ y,
                                                                const float* __restrict__ route_weights,
                                                                const int* __restrict__ slot_index, int E, int H, int slot_limit) {
    __shared__ int sl_slot[64];
    __shared__ float sl_w[64];
    __shared__ int sl_n;
    const int row = blockIdx.x, t = threadIdx.x;
    uint16_t* mrow = mixed + static_cast<size_t>(row) * H;
    for (int e0 = 0; e0 < E; e0 += 64) {
        if (t < 64) {
            const int e = e0 + t;
            const float w = e < E ? route_weights[static_cast<size_t>(row) * E + e] : 0.0f;
            const bool sel = w > 0.0f;
            // the table is filled for the pairs of the row lists only: a cell that does not name a row of y (a pair the
            // lists do not hold, or one cut off by the caller's row bound) is skipped
            int slot = sel ? slot_index[static_cast<size_t>(row) * E + e] : -1;
            if (static_cast<unsigned>(slot) >= static_cast<unsigned>(slot_limit)) slot = -1;     // also a negative cell
            const unsigned long long m = __ballot(sel);
            if (sel) {
                const int pos = __builtin_popcountll(m & ((1ull << t) - 1ull));
                sl_slot[pos] = slot;
                sl_w[pos] = UNIT ? 1.0f : w;
            }
            if (t == 0) sl_n = __builtin_popcountll(m);
        }
        __syncthreads();
        const int n = sl_n;
        if (n > 0) combine_rows(mrow, y, H, n, sl_slot, sl_w, t);
        __syncthreads();
    }
}

// slot_index[row, e] = offsets[e] + s for every entry s of expert e's list; other cells are left as they are
__global__ __launch_bounds__(kThreads) void k_slot_index(const int* __restrict__ counts, const int* __restrict__ offsets,
                                                         const int* __restrict__ row_indices, int rows, int E,
                                                         int* __restrict__ slot_index) {
    const int e = blockIdx.y;
    const int n = counts[e], base = offsets[e];
    for (int s = blockIdx.x * blockDim.x + threadIdx.x; s < n; s += gridDim.x * blockDim.x)
        slot_index[static_cast<size_t>(row_indices[static_cast<size_t>(e) * rows + s]) * E + e] = base + s;
}

// UNIT: every selected expert's row is added with factor 1 (the backward's scatter-add); the route weights
// then only say which experts selected the row.
template <bool UNIT, class YT = uint16_t>
__global__ __launch_bounds__(kThreads) void k_unpermute(uint16_t* __restrict__ mixed, const YT* __restrict__ y,
                                                        const float* __restrict__ route_weights,
                                                        const int* __restrict__ counts, const int* __restrict__ offsets,
                                                        const int* __restrict__ row_indices, int rows, int E, int H, int slot_limit) {
    __shared__ int sl_e[64];
    __shared__ int sl_slot[64];
    __shared__ float sl_w[64];
    __shared__ int sl_n;
    const int row = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
    uint16_t* mrow = mixed + static_cast<size_t>(row) * H;
    for (int e0 = 0; e0 < E; e0 += 64) {
        if (t < 64) {
            const int e = e0 + t;
            const float w = e < E ? route_weights[static_cast<size_t>(row) * E + e] : 0.0f;
            const bool sel = w > 0.0f;
            const unsigned long long m = __ballot(sel);
            if (sel) {
                const int pos = __builtin_popcountll(m & ((1ull << t) - 1ull));
                sl_e[pos] = e;
                sl_w[pos] = UNIT ? 1.0f : w;
            }
            if (t == 0) sl_n = __builtin_popcountll(m);
        }
        __syncthreads();
        const int n = sl_n;
        for (int i = wave; i < n; i += kThreads / 64) {
            const int e = sl_e[i];
            const int pos = wave_find_sorted(row_indices + static_cast<size_t>(e) * rows, counts[e], row, lane);
            // -1: not in the expert's list, or past the rows y holds: skipped
            if (lane == 0) sl_slot[i] = pos < 0 || offsets[e] + pos >= slot_limit ? -1 : offsets[e] + pos;
        }
        __syncthreads();
        if (n > 0) combine_rows(mrow, y, H, n, sl_slot, sl_w, t);
        __syncthreads();
    }
}

__device__ __forceinline__ void atomic_add_bf16(uint16_t* addr, float v) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(addr);
    auto* word = reinterpret_cast<unsigned int*>(a & ~static_cast<uintptr_t>(3));
    const unsigned shift = (a & 2) ? 16u : 0u;
    unsigned old = *word;
    while (true) {
        const unsigned assumed = old;
        const float cur = bf16_to_f32(static_cast<uint16_t>((assumed >> shift) & 0xffffu));
        const unsigned next = (assumed & ~(0xffffu << shift)) | (static_cast<unsigned>(f32_to_bf16(cur + v)) << shift);
        old = atomicCAS(word, assumed, next);
        if (old == assumed) return;
    }
}

// ---- grouped GELU expert bank, reference semantics, any shape --------------------------------
// mixed[row] += w * fc_out(gelu(fc_in(hidden[row]))) for every selected (expert,row): per-tensor descales, the
// exact-erf GELU output stays in fp32 (it is not re-quantised), products are accumulated in fp32, and the result is
// added to the bf16 output with a 32-bit compare-and-swap on the word holding it.  Shapes made of whole MFMA steps
// go to the matrix-core kernels below; this one takes everything else, with no alignment demands.
//
// One workgroup per (expert, R token rows); workgroups past an expert's row count leave at once.  The R hidden rows
// sit in LDS as fp32.  A projection is wave-parallel dot products: a wavefront takes C = 32 / R output columns at a
// time, lane l walks k = l, l + 64, ... (a weight row is contiguous in k, so the 64 lanes read 64 neighbouring
// elements of each of the C rows; the activations of the R rows come from LDS, one bank per lane), which leaves
// every lane with 32 partial sums; fold_values adds them over the 64 lanes in 32 exchanges instead of 32 x 6.
// The descales multiply the finished sums.  BF16: the bf16 sibling (moe_grouped_expert_forward_bf16): hidden and
// weights are bf16 (the byte pointers then address 2-byte elements), no descales.

// The sums of 32 per-lane values over the 64 lanes: each of five halving steps hands the half of the values this
// lane gives up to the lane across (xor 32, 16, 8, 4, 2) and adds what comes back to the half it keeps; one plain
// step (xor 1) finishes.  Value i ends in v[0] of lanes 2 i and 2 i + 1.
template <int N>
__device__ __forceinline__ void fold_values(float (&v)[32], int lane) {
    if constexpr (N > 1) {
        constexpr int half = N / 2;
        const bool upper = (lane & N) != 0;
#pragma unroll
        for (int i = 0; i < half; ++i) {
            const float send = upper ? v[i] : v[i + half];
            const float keep = upper ? v[i + half] : v[i];
            v[i] = keep + __shfl_xor(send, N, kWave);
        }
        fold_values<half>(v, lane);
    } else {
        v[0] += __shfl_xor(v[0], 1, kWave);
    }
}

// out(r, n, sum_k x[r][k] w[n][k]) for r < R and every n < N, called by one lane per (r, n); x in LDS [R][K]
template <int R, class Elem, class Out>
__device__ __forceinline__ void project_rows(const float* x, int K, int N, Elem&& weight, Out&& out) {
    constexpr int C = 32 / R;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int n0 = wave * C; n0 < N; n0 += (kThreads / 64) * C) {
        float v[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = 0.0f;
        size_t wrow[C];
#pragma unroll
        for (int c = 0; c < C; ++c) wrow[c] = static_cast<size_t>(min(n0 + c, N - 1)) * K;
        for (int k = lane; k < K; k += 64) {
            float xv[R];
#pragma unroll
            for (int r = 0; r < R; ++r) xv[r] = x[r * K + k];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float wv = weight(wrow[c] + k);
#pragma unroll
                for (int r = 0; r < R; ++r) v[r * C + c] = __builtin_fmaf(xv[r], wv, v[r * C + c]);
            }
        }
        fold_values<32>(v, lane);
        const int idx = lane >> 1, r = idx / C, c = idx % C;
        if ((lane & 1) == 0 && n0 + c < N) out(r, n0 + c, v[0]);
    }
}

template <bool BF16, int R>
__global__ __launch_bounds__(kThreads) void k_grouped_gelu_wave(const uint8_t* __restrict__ hidden, const float* __restrict__ fcin_descale,
                                                                int fcin_is_e5m2, const float* __restrict__ route_weights,
                                                                const int* __restrict__ counts, const int* __restrict__ row_indices,
                                                                const uint8_t* __restrict__ fc_in_w, const float* __restrict__ fc_in_descale,
                                                                const uint8_t* __restrict__ fc_out_w, const float* __restrict__ fc_out_descale,
                                                                uint16_t* __restrict__ mixed, int rows, int H, int Ie, int E,
                                                                int tiles_per_expert) {
    extern __shared__ float sh[];
    float* xs = sh;                        // [R][H]: the tile's hidden rows, decoded, not yet descaled
    float* act = sh + R * H;               // [R][Ie]: GELU output
    const int e = blockIdx.x / tiles_per_expert, tile = blockIdx.x % tiles_per_expert;
    const int first = tile * R, n_active = counts[e];
    if (first >= n_active) return;
    const int n_rows = min(R, n_active - first);
    const int* my_rows = row_indices + static_cast<size_t>(e) * rows + first;
    constexpr int kElem = BF16 ? 2 : 1;
    const uint8_t* w_in = fc_in_w + static_cast<size_t>(e) * H * Ie * kElem;
    const uint8_t* w_out = fc_out_w + static_cast<size_t>(e) * Ie * H * kElem;
    const float s_in = BF16 ? 1.0f : *fcin_descale * *fc_in_descale, s_out = BF16 ? 1.0f : *fc_out_descale;
    auto element = [](const uint8_t* p, size_t i, bool e5m2) {
        if constexpr (BF16) return bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
        else return e5m2 ? e5m2_to_f32(p[i]) : e4m3_to_f32(p[i]);
    };
    for (int i = threadIdx.x; i < R * H; i += kThreads) {
        const int r = i / H, k = i - r * H;
        xs[i] = r < n_rows ? element(hidden, static_cast<size_t>(my_rows[r]) * H + k, fcin_is_e5m2 != 0) : 0.0f;
    }
    __syncthreads();
    project_rows<R>(xs, H, Ie, [&](size_t i) { return element(w_in, i, false); },
                    [&](int r, int j, float sum) {
                        // the bf16 sibling parks the activation as bf16 (kernels/moe.cu:845); the FP8 kernel keeps fp32 (:1031)
                        const float g = gelu_fwd(sum * s_in);
                        act[r * Ie + j] = BF16 ? bf16_to_f32(f32_to_bf16(g)) : g;
                    });
    __syncthreads();
    project_rows<R>(act, Ie, H, [&](size_t i) { return element(w_out, i, false); },
                    [&](int r, int h, float sum) {
                        if (r >= n_rows) return;
                        const int row = my_rows[r];
                        atomic_add_bf16(mixed + static_cast<size_t>(row) * H + h, route_weights[static_cast<size_t>(row) * E + e] * (sum * s_out));
                    });
}

// R token rows per workgroup: the most (of 8, 4, 2, 1) whose fp32 hidden rows and GELU rows fit the LDS
template <bool BF16>
int launch_grouped_gelu_wave(const uint8_t* hidden, const float* fcin_descale, int fcin_is_e5m2, const float* route_weights,
                             const int* counts, const int* row_indices, const uint8_t* fc_in_w, const float* fc_in_descale,
                             const uint8_t* fc_out_w, const float* fc_out_descale, uint16_t* mixed, int rows, int H, int Ie, int E,
                             hipStream_t st) {
    const size_t per_row = sizeof(float) * (static_cast<size_t>(H) + Ie);
    auto go = [&](auto rc) {
        constexpr int R = decltype(rc)::value;
        static std::once_flag once;
        static hipError_t attr_err = hipSuccess;
        std::call_once(once, [] {
            attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_grouped_gelu_wave<BF16, R>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        });
        if (attr_err != hipSuccess) return static_cast<int>(attr_err);
        const int tiles_per_expert = (rows + R - 1) / R;
        if (static_cast<long long>(E) * tiles_per_expert >= (1LL << 31)) return static_cast<int>(CF_ERR_UNSUPPORTED);
        k_grouped_gelu_wave<BF16, R><<<E * tiles_per_expert, kThreads, R * per_row, st>>>(
            hidden, fcin_descale, fcin_is_e5m2, route_weights, counts, row_indices, fc_in_w, fc_in_descale, fc_out_w, fc_out_descale,
            mixed, rows, H, Ie, E, tiles_per_expert);
        return launch_status();
    };
    constexpr size_t kLdsBytes = 160 * 1024;
    if (8 * per_row <= kLdsBytes) return go(std::integral_constant<int, 8>{});
    if (4 * per_row <= kLdsBytes) return go(std::integral_constant<int, 4>{});
    if (2 * per_row <= kLdsBytes) return go(std::integral_constant<int, 2>{});
    if (per_row <= kLdsBytes) return go(std::integral_constant<int, 1>{});
    return static_cast<int>(CF_ERR_UNSUPPORTED);
}

// ---- the same bank on the matrix cores -----------------------------------------------------------
// Same arithmetic contract (GELU output kept beyond bf16, nothing re-quantised, compare-and-swap accumulation), for
// H % 128 == 0 and Ie % 64 == 0.  One workgroup per (expert, 16 rows), eight wavefronts:
//   fc_in   v_mfma_f32_16x16x128_f8f6f4 on the fp8 bytes as they are (products of fp8 values are exact in the fp32
//           accumulator; the two per-tensor descales multiply the sum).  The 16 hidden rows sit in LDS, weight rows
//           come from L2 as 32-byte runs per lane.
//   GELU    in fp32 on the accumulator, split into a bf16 head and a bf16 remainder (together 16 significand bits,
//           relative error 2^-17) and parked in LDS.
//   fc_out  v_mfma_f32_16x16x32_bf16 twice per step (head and remainder) against the E4M3 weights widened to bf16,
//           which is exact.  A lane fetches 32 weight bytes at once (the four lane groups cover a whole 128-byte line
//           of a weight row) and uses them as four k-blocks of 8; the activation reads follow the same order, and a
//           sum does not care which k a lane group holds.
// Weights go to the "A" side, so a lane ends with 4 neighbouring output columns of one token row.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
constexpr int kMfmaRows = 16;

__device__ __forceinline__ v8bf e4m3x8_to_bf16(uint32_t a, uint32_t b) {
    const f32x2_t p0 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(a), false), p1 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(a), true);
    const f32x2_t p2 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(b), false), p3 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(b), true);
    // the upper halves of the two floats, side by side (bytes 2,3 of the first, then 2,3 of the second)
    auto pair = [](f32x2_t p) { return __builtin_amdgcn_perm(__float_as_uint(p[1]), __float_as_uint(p[0]), 0x07060302u); };
    const v4u w = {pair(p0), pair(p1), pair(p2), pair(p3)};
    return __builtin_bit_cast(v8bf, w);
}

// four neighbouring bf16 values += v[0..3], one rounding each, by a 64-bit compare-and-swap; `old` is a value read
// from the address earlier (a stale one only costs a second round)
__device__ __forceinline__ unsigned long long add_bf16x4(unsigned long long cur, const float* v) {
    const unsigned lo = static_cast<unsigned>(cur), hi = static_cast<unsigned>(cur >> 32);
    return static_cast<unsigned long long>(pack_bf16x2(bf16_lo(lo) + v[0], bf16_hi(lo) + v[1])) |
           (static_cast<unsigned long long>(pack_bf16x2(bf16_lo(hi) + v[2], bf16_hi(hi) + v[3])) << 32);
}
__device__ __forceinline__ void atomic_add_bf16x4(unsigned long long* quad, unsigned long long old, const float* v) {
    while (true) {
        const unsigned long long assumed = old;
        old = atomicCAS(quad, assumed, add_bf16x4(assumed, v));
        if (old == assumed) return;
    }
}

constexpr int kMfmaThreads = 512;      // eight wavefronts: two per SIMD, so one's weight fetches hide behind the other's MFMAs
constexpr int kXcdCount = 8;
constexpr int kMfmaOutDepth = 4;       // the same per output block in fc_out, which carries kMfmaBlocks of them
constexpr int kMfmaBlocks = 2;         // output blocks a wavefront carries through one pass over k
constexpr int kMfmaDepth = 4;          // weight fetches a wavefront keeps in flight ahead of its MFMAs

template <bool E5M2>
__global__ __launch_bounds__(kMfmaThreads) void k_grouped_gelu_fp8_mfma(const uint8_t* __restrict__ hidden, const float* __restrict__ fcin_descale,
                                                                        const float* __restrict__ route_weights, const int* __restrict__ counts,
                                                                        const int* __restrict__ row_indices, const uint8_t* __restrict__ fc_in_w,
                                                                        const float* __restrict__ fc_in_descale, const uint8_t* __restrict__ fc_out_w,
                                                                        const float* __restrict__ fc_out_descale, uint16_t* __restrict__ mixed,
                                                                        int rows, int H, int Ie, int E, int tiles_per_expert) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kWaves = kMfmaThreads / 64;
    const int hs = H + 16;                          // hidden row stride in bytes: neighbouring rows 16 bytes apart in the banks
    const int as = Ie + 8;                          // activation row stride in elements, likewise
    uint8_t* sh_hidden = smem;                                                        // [16][hs] fp8
    uint16_t* sh_hi = reinterpret_cast<uint16_t*>(smem + kMfmaRows * hs);             // [16][as] bf16 head of gelu
    uint16_t* sh_lo = sh_hi + kMfmaRows * as;                                         // [16][as] bf16 remainder
    // workgroups go round the 8 XCDs in turn: give each XCD whole experts, so one expert's weights (re-read by every
    // 16-row tile) are served by that XCD's L2
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int e = (slot / tiles_per_expert) * kXcdCount + xcd, tile = slot % tiles_per_expert;
    if (e >= E) return;
    const int first = tile * kMfmaRows, n_active = counts[e];
    if (first >= n_active) return;
    const int n_rows = min(kMfmaRows, n_active - first);
    const int* my_rows = row_indices + static_cast<size_t>(e) * rows + first;
    const uint8_t* w_in = fc_in_w + static_cast<size_t>(e) * H * Ie;
    const uint8_t* w_out = fc_out_w + static_cast<size_t>(e) * Ie * H;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, t = lane & 15, g = lane >> 4;

    // the tile's hidden rows (rows past the list's end repeat its last one; their results are dropped)
    const int vec_per_row = H / 16;
    for (int i = threadIdx.x; i < kMfmaRows * vec_per_row; i += kMfmaThreads) {
        const int r = i / vec_per_row, c = i % vec_per_row;
        const int src = my_rows[min(r, n_rows - 1)];
        *reinterpret_cast<uint4*>(sh_hidden + r * hs + c * 16) =
            *reinterpret_cast<const uint4*>(hidden + static_cast<size_t>(src) * H + c * 16);
    }
    __syncthreads();

    const float s_in = *fcin_descale * *fc_in_descale;
    const int in_steps = H / 128;
    for (int n0 = wave * 16; n0 < Ie; n0 += kWaves * 16) {
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
        const uint8_t* wr = w_in + static_cast<size_t>(n0 + t) * H + 32 * g;
        const uint8_t* hr = sh_hidden + t * hs + 32 * g;
        uint4 w0[kMfmaDepth], w1[kMfmaDepth];
#pragma unroll
        for (int j = 0; j < kMfmaDepth; ++j)
            if (j < in_steps) {
                w0[j] = *reinterpret_cast<const uint4*>(wr + j * 128);
                w1[j] = *reinterpret_cast<const uint4*>(wr + j * 128 + 16);
            }
        for (int s0 = 0; s0 < in_steps; s0 += kMfmaDepth) {
#pragma unroll
            for (int j = 0; j < kMfmaDepth; ++j) {
                const int st = s0 + j;
                if (st < in_steps) {
                    const uint4 x0 = *reinterpret_cast<const uint4*>(hr + st * 128), x1 = *reinterpret_cast<const uint4*>(hr + st * 128 + 16);
                    const v8i a = {(int)w0[j].x, (int)w0[j].y, (int)w0[j].z, (int)w0[j].w, (int)w1[j].x, (int)w1[j].y, (int)w1[j].z, (int)w1[j].w};
                    const v8i b = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
                    if (st + kMfmaDepth < in_steps) {
                        w0[j] = *reinterpret_cast<const uint4*>(wr + (st + kMfmaDepth) * 128);
                        w1[j] = *reinterpret_cast<const uint4*>(wr + (st + kMfmaDepth) * 128 + 16);
                    }
                    acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc, 0 /* weights E4M3 */, E5M2 ? 1 : 0, 0, 0, 0, 0);
                }
            }
        }
        // this lane: token row t, columns n0 + 4g .. + 3
        uint32_t hb[4], lb[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = acc[r] * s_in;
            const float act = gelu_fwd(v);
            hb[r] = __float_as_uint(act) & 0xffff0000u;
            lb[r] = f32_to_bf16(act - __uint_as_float(hb[r]));
        }
        const int at = t * as + n0 + 4 * g;
        *reinterpret_cast<uint2*>(sh_hi + at) = make_uint2((hb[0] >> 16) | hb[1], (hb[2] >> 16) | hb[3]);
        *reinterpret_cast<uint2*>(sh_lo + at) = make_uint2(lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16));
    }
    __syncthreads();

    const float d_wout = *fc_out_descale;
    const int out_steps = Ie / 128;                 // whole 128-byte lines of a weight row; Ie % 128 == 64 leaves half a line
    const int out_tail = out_steps * 128;
    const bool live = t < n_rows;
    const int row = live ? my_rows[t] : 0;
    const float rw = live ? route_weights[static_cast<size_t>(row) * E + e] : 0.0f;
    const uint16_t* ah = sh_hi + t * as;
    const uint16_t* al = sh_lo + t * as;
    // kMfmaBlocks output blocks per pass share every activation read from LDS (the LDS port, not the MFMA, is what a
    // pass with one block waits for).  A block past the end repeats the last one and is not written.
    for (int h0 = wave * 16; h0 < H; h0 += kWaves * 16 * kMfmaBlocks) {
        v4f acc_hi[kMfmaBlocks], acc_lo[kMfmaBlocks];
        const uint8_t* wrow[kMfmaBlocks];
        unsigned long long* quad[kMfmaBlocks];
        unsigned long long before[kMfmaBlocks];
        uint4 wa[kMfmaBlocks][kMfmaOutDepth], wb[kMfmaBlocks][kMfmaOutDepth], wt[kMfmaBlocks];
#pragma unroll
        for (int b = 0; b < kMfmaBlocks; ++b) {
            const int hb = min(h0 + b * kWaves * 16, H - 16);
            acc_hi[b] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            acc_lo[b] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            // the four output values this lane will add to, fetched now so the read is not waited for after the MFMAs
            quad[b] = reinterpret_cast<unsigned long long*>(mixed + static_cast<size_t>(row) * H + hb + 4 * g);
            before[b] = live ? __builtin_nontemporal_load(quad[b]) : 0ull;
            wrow[b] = w_out + static_cast<size_t>(hb + t) * Ie;
#pragma unroll
            for (int j = 0; j < kMfmaOutDepth; ++j)
                if (j < out_steps) {                                                // step s: k = 128 s + 32 g .. + 31
                    wa[b][j] = *reinterpret_cast<const uint4*>(wrow[b] + 32 * g + j * 128);
                    wb[b][j] = *reinterpret_cast<const uint4*>(wrow[b] + 32 * g + j * 128 + 16);
                }
            wt[b] = make_uint4(0u, 0u, 0u, 0u);
            if (Ie & 64) wt[b] = *reinterpret_cast<const uint4*>(wrow[b] + out_tail + 16 * g);   // half line: k = tail + 16 g .. + 15
        }
        // 8 weights of this lane's k run, per block, against the head and the remainder of the same 8 activations
        auto mm = [&](const uint32_t (&x)[kMfmaBlocks], const uint32_t (&y)[kMfmaBlocks], int k) {
            const v8bf hv = *reinterpret_cast<const v8bf*>(ah + k), lv = *reinterpret_cast<const v8bf*>(al + k);
#pragma unroll
            for (int b = 0; b < kMfmaBlocks; ++b) {
                const v8bf wv = e4m3x8_to_bf16(x[b], y[b]);
                acc_hi[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, hv, acc_hi[b], 0, 0, 0);
                acc_lo[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, lv, acc_lo[b], 0, 0, 0);
            }
        };
        for (int s0 = 0; s0 < out_steps; s0 += kMfmaOutDepth) {
#pragma unroll
            for (int j = 0; j < kMfmaOutDepth; ++j) {
                const int st = s0 + j;
                if (st < out_steps) {
                    uint32_t c[8][kMfmaBlocks];
#pragma unroll
                    for (int b = 0; b < kMfmaBlocks; ++b) {
                        c[0][b] = wa[b][j].x; c[1][b] = wa[b][j].y; c[2][b] = wa[b][j].z; c[3][b] = wa[b][j].w;
                        c[4][b] = wb[b][j].x; c[5][b] = wb[b][j].y; c[6][b] = wb[b][j].z; c[7][b] = wb[b][j].w;
                        if (st + kMfmaOutDepth < out_steps) {
                            wa[b][j] = *reinterpret_cast<const uint4*>(wrow[b] + 32 * g + (st + kMfmaOutDepth) * 128);
                            wb[b][j] = *reinterpret_cast<const uint4*>(wrow[b] + 32 * g + (st + kMfmaOutDepth) * 128 + 16);
                        }
                    }
                    const int k = st * 128 + 32 * g;
                    mm(c[0], c[1], k);
                    mm(c[2], c[3], k + 8);
                    mm(c[4], c[5], k + 16);
                    mm(c[6], c[7], k + 24);
                }
            }
        }
        if (Ie & 64) {
            uint32_t c[4][kMfmaBlocks];
#pragma unroll
            for (int b = 0; b < kMfmaBlocks; ++b) { c[0][b] = wt[b].x; c[1][b] = wt[b].y; c[2][b] = wt[b].z; c[3][b] = wt[b].w; }
            mm(c[0], c[1], out_tail + 16 * g);
            mm(c[2], c[3], out_tail + 16 * g + 8);
        }
#pragma unroll
        for (int b = 0; b < kMfmaBlocks; ++b) {
            if (live && h0 + b * kWaves * 16 < H) {
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = rw * ((acc_hi[b][r] + acc_lo[b][r]) * d_wout);
                atomic_add_bf16x4(quad[b], before[b], v);
            }
        }
    }
}

// ---- 32-row form ------------------------------------------------------------------------------------
// The 16-row kernel above re-reads its expert's weights once per 16 rows, and that traffic through the L2s is what
// it waits for.  This form takes 32 rows per workgroup (two groups of 16 token rows against every weight fetch) and
// still keeps the GELU output at 4 bytes per element in LDS by walking Ie in chunks: fc_in + GELU for a chunk of
// columns, then that chunk's share of fc_out added into accumulators that stay in registers across chunks: a
// wavefront owns the output blocks wave, wave + 8, ... (H / 128 of them, at most kWideBlocks: H <= 2048), two
// accumulators each.  Blocks are walked in pairs so an activation read from LDS feeds two blocks.  One rounding
// per (row, expert) as before: the compare-and-swap comes after the last chunk.
constexpr int kWideRows = 32;
constexpr int kWideBlocks = 16;
constexpr int kWideDepth = 2;

template <bool E5M2>
__global__ __launch_bounds__(kMfmaThreads) void k_grouped_gelu_fp8_mfma32(const uint8_t* __restrict__ hidden, const float* __restrict__ fcin_descale,
                                                                          const float* __restrict__ route_weights, const int* __restrict__ counts,
                                                                          const int* __restrict__ row_indices, const uint8_t* __restrict__ fc_in_w,
                                                                          const float* __restrict__ fc_in_descale, const uint8_t* __restrict__ fc_out_w,
                                                                          const float* __restrict__ fc_out_descale, uint16_t* __restrict__ mixed,
                                                                          int rows, int H, int Ie, int E, int tiles_per_expert, int chunk) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kWaves = kMfmaThreads / 64;
    const int hs = H + 16;                          // hidden row stride in bytes
    const int as = chunk + 8;                       // activation row stride in elements
    uint8_t* sh_hidden = smem;                                                        // [32][hs] fp8
    uint16_t* sh_hi = reinterpret_cast<uint16_t*>(smem + kWideRows * hs);             // [32][as] bf16 head of gelu
    uint16_t* sh_lo = sh_hi + kWideRows * as;                                         // [32][as] bf16 remainder
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int e = (slot / tiles_per_expert) * kXcdCount + xcd, tile = slot % tiles_per_expert;
    if (e >= E) return;
    const int first = tile * kWideRows, n_active = counts[e];
    if (first >= n_active) return;
    const int n_rows = min(kWideRows, n_active - first);
    const int* my_rows = row_indices + static_cast<size_t>(e) * rows + first;
    const uint8_t* w_in = fc_in_w + static_cast<size_t>(e) * H * Ie;
    const uint8_t* w_out = fc_out_w + static_cast<size_t>(e) * Ie * H;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, t = lane & 15, g = lane >> 4;

    const int vec_per_row = H / 16;
    for (int i = threadIdx.x; i < kWideRows * vec_per_row; i += kMfmaThreads) {
        const int r = i / vec_per_row, c = i % vec_per_row;
        const int src = my_rows[min(r, n_rows - 1)];
        *reinterpret_cast<uint4*>(sh_hidden + r * hs + c * 16) =
            *reinterpret_cast<const uint4*>(hidden + static_cast<size_t>(src) * H + c * 16);
    }
    __syncthreads();

    const float s_in = *fcin_descale * *fc_in_descale;
    const int in_steps = H / 128;
    const int nblk = H / 128;                       // output blocks of this wavefront
    v4f acc[kWideBlocks][2];
#pragma unroll
    for (int b = 0; b < kWideBlocks; ++b) {
        acc[b][0] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        acc[b][1] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }

    for (int c0 = 0; c0 < Ie; c0 += chunk) {
        const int cw = min(chunk, Ie - c0);         // a multiple of 64
        // ---- fc_in + GELU for columns c0 .. c0 + cw - 1 ----
        for (int n0 = wave * 16; n0 < cw; n0 += kWaves * 16) {
            v4f a0 = {0.0f, 0.0f, 0.0f, 0.0f}, a1 = {0.0f, 0.0f, 0.0f, 0.0f};
            const uint8_t* wr = w_in + static_cast<size_t>(c0 + n0 + t) * H + 32 * g;
            const uint8_t* hr0 = sh_hidden + t * hs + 32 * g;
            const uint8_t* hr1 = hr0 + 16 * hs;
            uint4 w0[kWideDepth], w1[kWideDepth];
#pragma unroll
            for (int j = 0; j < kWideDepth; ++j)
                if (j < in_steps) {
                    w0[j] = *reinterpret_cast<const uint4*>(wr + j * 128);
                    w1[j] = *reinterpret_cast<const uint4*>(wr + j * 128 + 16);
                }
            for (int s0 = 0; s0 < in_steps; s0 += kWideDepth) {
#pragma unroll
                for (int j = 0; j < kWideDepth; ++j) {
                    const int st = s0 + j;
                    if (st < in_steps) {
                        const v8i a = {(int)w0[j].x, (int)w0[j].y, (int)w0[j].z, (int)w0[j].w, (int)w1[j].x, (int)w1[j].y, (int)w1[j].z, (int)w1[j].w};
                        if (st + kWideDepth < in_steps) {
                            w0[j] = *reinterpret_cast<const uint4*>(wr + (st + kWideDepth) * 128);
                            w1[j] = *reinterpret_cast<const uint4*>(wr + (st + kWideDepth) * 128 + 16);
                        }
                        const uint4 x0 = *reinterpret_cast<const uint4*>(hr0 + st * 128), x1 = *reinterpret_cast<const uint4*>(hr0 + st * 128 + 16);
                        const uint4 y0 = *reinterpret_cast<const uint4*>(hr1 + st * 128), y1 = *reinterpret_cast<const uint4*>(hr1 + st * 128 + 16);
                        const v8i b0 = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
                        const v8i b1 = {(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
                        a0 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b0, a0, 0, E5M2 ? 1 : 0, 0, 0, 0, 0);
                        a1 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b1, a1, 0, E5M2 ? 1 : 0, 0, 0, 0, 0);
                    }
                }
            }
            // this lane: token rows t and 16 + t, columns c0 + n0 + 4g .. + 3
#pragma unroll
            for (int tg = 0; tg < 2; ++tg) {
                uint32_t hb[4], lb[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float act = gelu_fwd((tg ? a1[r] : a0[r]) * s_in);
                    hb[r] = __float_as_uint(act) & 0xffff0000u;
                    lb[r] = f32_to_bf16(act - __uint_as_float(hb[r]));
                }
                const int at = (tg * 16 + t) * as + n0 + 4 * g;
                *reinterpret_cast<uint2*>(sh_hi + at) = make_uint2((hb[0] >> 16) | hb[1], (hb[2] >> 16) | hb[3]);
                *reinterpret_cast<uint2*>(sh_lo + at) = make_uint2(lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16));
            }
        }
        __syncthreads();

        // ---- this chunk's share of fc_out ----
        const int steps = cw / 128, tail = steps * 128;     // whole 128-byte runs of the chunk; cw % 128 == 64 leaves half a run
        const uint32_t lane_row = static_cast<uint32_t>(wave * 16 + t) * static_cast<uint32_t>(Ie);
        const uint16_t* ah0 = sh_hi + t * as;
        const uint16_t* al0 = sh_lo + t * as;
        const uint16_t* ah1 = ah0 + 16 * as;
        const uint16_t* al1 = al0 + 16 * as;
#pragma unroll
        for (int bp = 0; bp < kWideBlocks; bp += 2) {
            if (bp < nblk) {
                // rows of the two blocks' weights (the second repeats the first where nblk is odd; its sums are not used)
                // uniform base + 32-bit lane offsets: no 64-bit per-lane addresses to keep alive across the pairs
                const int bq = bp + 1 < nblk ? bp + 1 : bp;
                const uint8_t* wbase = w_out + c0;
                const uint32_t oA = lane_row + static_cast<uint32_t>(kWaves * 16 * bp) * static_cast<uint32_t>(Ie);
                const uint32_t oB = lane_row + static_cast<uint32_t>(kWaves * 16 * bq) * static_cast<uint32_t>(Ie);
                auto ldw = [&](uint32_t off) { return *reinterpret_cast<const uint4*>(wbase + off); };
                v4f pA0 = acc[bp][0], pA1 = acc[bp][1], pB0 = acc[bp + 1][0], pB1 = acc[bp + 1][1];
                auto mm = [&](uint32_t xa, uint32_t ya, uint32_t xb, uint32_t yb, int k) {
                    const v8bf wa = e4m3x8_to_bf16(xa, ya), wb = e4m3x8_to_bf16(xb, yb);
                    const v8bf h0 = *reinterpret_cast<const v8bf*>(ah0 + k), h1 = *reinterpret_cast<const v8bf*>(ah1 + k);
                    const v8bf l0 = *reinterpret_cast<const v8bf*>(al0 + k), l1 = *reinterpret_cast<const v8bf*>(al1 + k);
                    pA0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, h0, pA0, 0, 0, 0);
                    pA1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, h1, pA1, 0, 0, 0);
                    pB0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, h0, pB0, 0, 0, 0);
                    pB1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, h1, pB1, 0, 0, 0);
                    pA0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, l0, pA0, 0, 0, 0);
                    pA1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, l1, pA1, 0, 0, 0);
                    pB0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, l0, pB0, 0, 0, 0);
                    pB1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, l1, pB1, 0, 0, 0);
                };
                uint4 a0[kWideDepth], a1[kWideDepth], b0[kWideDepth], b1[kWideDepth];
#pragma unroll
                for (int j = 0; j < kWideDepth; ++j)
                    if (j < steps) {                                                // step s: k = 128 s + 32 g .. + 31 of the chunk
                        a0[j] = ldw(oA + 32 * g + j * 128);
                        a1[j] = ldw(oA + 32 * g + j * 128 + 16);
                        b0[j] = ldw(oB + 32 * g + j * 128);
                        b1[j] = ldw(oB + 32 * g + j * 128 + 16);
                    }
                for (int s0 = 0; s0 < steps; s0 += kWideDepth) {
#pragma unroll
                    for (int j = 0; j < kWideDepth; ++j) {
                        const int st = s0 + j;
                        if (st < steps) {
                            const uint4 ca0 = a0[j], ca1 = a1[j], cb0 = b0[j], cb1 = b1[j];
                            if (st + kWideDepth < steps) {
                                a0[j] = ldw(oA + 32 * g + (st + kWideDepth) * 128);
                                a1[j] = ldw(oA + 32 * g + (st + kWideDepth) * 128 + 16);
                                b0[j] = ldw(oB + 32 * g + (st + kWideDepth) * 128);
                                b1[j] = ldw(oB + 32 * g + (st + kWideDepth) * 128 + 16);
                            }
                            const int k = st * 128 + 32 * g;
                            mm(ca0.x, ca0.y, cb0.x, cb0.y, k);
                            mm(ca0.z, ca0.w, cb0.z, cb0.w, k + 8);
                            mm(ca1.x, ca1.y, cb1.x, cb1.y, k + 16);
                            mm(ca1.z, ca1.w, cb1.z, cb1.w, k + 24);
                        }
                    }
                }
                if (cw & 64) {                                                      // half run: k = tail + 16 g .. + 15
                    const uint4 ta = ldw(oA + tail + 16 * g);
                    const uint4 tb = ldw(oB + tail + 16 * g);
                    mm(ta.x, ta.y, tb.x, tb.y, tail + 16 * g);
                    mm(ta.z, ta.w, tb.z, tb.w, tail + 16 * g + 8);
                }
                acc[bp][0] = pA0; acc[bp][1] = pA1; acc[bp + 1][0] = pB0; acc[bp + 1][1] = pB1;
            }
        }
        __syncthreads();                            // the next chunk overwrites the activations
    }

    // ---- one compare-and-swap per (token row, 4 output columns), four in flight at a time ----
    const float d_wout = *fc_out_descale;
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
        const int r = tg * 16 + t;
        const bool live = r < n_rows;
        const int row = live ? my_rows[r] : 0;
        const float rw = live ? route_weights[static_cast<size_t>(row) * E + e] : 0.0f;
        uint16_t* mrow = mixed + static_cast<size_t>(row) * H + 4 * g + wave * 16;
#pragma unroll
        for (int b0 = 0; b0 < kWideBlocks; b0 += 4) {
            if (b0 < nblk && live) {
                unsigned long long before[4], got[4];
                float v[4][4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (b0 + i < nblk)
                        before[i] = __builtin_nontemporal_load(reinterpret_cast<unsigned long long*>(mrow + (b0 + i) * kWaves * 16));
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (b0 + i < nblk) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) v[i][q] = rw * (acc[b0 + i][tg][q] * d_wout);
                        got[i] = atomicCAS(reinterpret_cast<unsigned long long*>(mrow + (b0 + i) * kWaves * 16), before[i],
                                           add_bf16x4(before[i], v[i]));
                    }
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (b0 + i < nblk && got[i] != before[i])                     // lost a race: redo from the value found
                        atomic_add_bf16x4(reinterpret_cast<unsigned long long*>(mrow + (b0 + i) * kWaves * 16), got[i], v[i]);
            }
            __builtin_amdgcn_sched_barrier(0);      // keeps the groups apart: their loads hoisted together would not fit the registers
        }
    }
}

// ---- the bf16 sibling on the matrix cores -------------------------------------------------------------
// moe_grouped_expert_forward_bf16 in the 16-row form above: both projections are v_mfma_f32_16x16x32_bf16 (products
// of two bf16 values are exact in the fp32 accumulator); the GELU output is rounded to bf16 before fc_out, as the
// reference kernel parks it (sh_fcin[j] = __float2bfloat16(g), kernels/moe.cu:845).
// A 128-byte run of a weight row is 64 elements: a lane fetches 32 bytes = two k-blocks of 8.  H % 64 == 0,
// Ie % 64 == 0.
__global__ __launch_bounds__(kMfmaThreads) void k_grouped_gelu_bf16_mfma(const uint16_t* __restrict__ hidden, const float* __restrict__ route_weights,
                                                                         const int* __restrict__ counts, const int* __restrict__ row_indices,
                                                                         const uint16_t* __restrict__ fc_in_w, const uint16_t* __restrict__ fc_out_w,
                                                                         uint16_t* __restrict__ mixed, int rows, int H, int Ie, int E,
                                                                         int tiles_per_expert) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kWaves = kMfmaThreads / 64;
    const int hs = H + 8;                           // row strides in elements: neighbouring rows 16 bytes apart in the banks
    const int as = Ie + 8;
    uint16_t* sh_hidden = reinterpret_cast<uint16_t*>(smem);                          // [16][hs]
    uint16_t* sh_hi = sh_hidden + kMfmaRows * hs;                                     // [16][as] bf16(gelu)
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int e = (slot / tiles_per_expert) * kXcdCount + xcd, tile = slot % tiles_per_expert;
    if (e >= E) return;
    const int first = tile * kMfmaRows, n_active = counts[e];
    if (first >= n_active) return;
    const int n_rows = min(kMfmaRows, n_active - first);
    const int* my_rows = row_indices + static_cast<size_t>(e) * rows + first;
    const uint16_t* w_in = fc_in_w + static_cast<size_t>(e) * H * Ie;
    const uint16_t* w_out = fc_out_w + static_cast<size_t>(e) * Ie * H;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, t = lane & 15, g = lane >> 4;

    const int vec_per_row = H / 8;
    for (int i = threadIdx.x; i < kMfmaRows * vec_per_row; i += kMfmaThreads) {
        const int r = i / vec_per_row, c = i % vec_per_row;
        const int src = my_rows[min(r, n_rows - 1)];
        *reinterpret_cast<uint4*>(sh_hidden + r * hs + c * 8) =
            *reinterpret_cast<const uint4*>(hidden + static_cast<size_t>(src) * H + c * 8);
    }
    __syncthreads();

    // one projection's inner product for a block of 16 weight rows: step s covers k = 64 s + 16 g .. + 15 of this lane
    auto load2 = [](const uint16_t* p, v8bf& a, v8bf& b) {
        a = *reinterpret_cast<const v8bf*>(p);
        b = *reinterpret_cast<const v8bf*>(p + 8);
    };
    const int in_steps = H / 64;
    for (int n0 = wave * 16; n0 < Ie; n0 += kWaves * 16) {
        v4f acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
        const uint16_t* wr = w_in + static_cast<size_t>(n0 + t) * H + 16 * g;
        const uint16_t* hr = sh_hidden + t * hs + 16 * g;
        v8bf wa[kMfmaDepth], wb[kMfmaDepth];
#pragma unroll
        for (int j = 0; j < kMfmaDepth; ++j)
            if (j < in_steps) load2(wr + j * 64, wa[j], wb[j]);
        for (int s0 = 0; s0 < in_steps; s0 += kMfmaDepth) {
#pragma unroll
            for (int j = 0; j < kMfmaDepth; ++j) {
                const int st = s0 + j;
                if (st < in_steps) {
                    const v8bf ca = wa[j], cb = wb[j];
                    if (st + kMfmaDepth < in_steps) load2(wr + (st + kMfmaDepth) * 64, wa[j], wb[j]);
                    v8bf xa, xb;
                    load2(hr + st * 64, xa, xb);
                    acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ca, xa, acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cb, xb, acc1, 0, 0, 0);
                }
            }
        }
        uint32_t hb[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) hb[r] = f32_to_bf16(gelu_fwd(acc0[r] + acc1[r]));
        const int at = t * as + n0 + 4 * g;
        *reinterpret_cast<uint2*>(sh_hi + at) = make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
    }
    __syncthreads();

    const int out_steps = Ie / 64;
    const bool live = t < n_rows;
    const int row = live ? my_rows[t] : 0;
    const float rw = live ? route_weights[static_cast<size_t>(row) * E + e] : 0.0f;
    const uint16_t* ah = sh_hi + t * as + 16 * g;
    for (int h0 = wave * 16; h0 < H; h0 += kWaves * 16) {
        v4f acc_hi = {0.0f, 0.0f, 0.0f, 0.0f}, acc_lo = {0.0f, 0.0f, 0.0f, 0.0f};
        auto* quad = reinterpret_cast<unsigned long long*>(mixed + static_cast<size_t>(row) * H + h0 + 4 * g);
        const unsigned long long before = live ? __builtin_nontemporal_load(quad) : 0ull;
        const uint16_t* wr = w_out + static_cast<size_t>(h0 + t) * Ie + 16 * g;
        v8bf wa[kMfmaDepth], wb[kMfmaDepth];
#pragma unroll
        for (int j = 0; j < kMfmaDepth; ++j)
            if (j < out_steps) load2(wr + j * 64, wa[j], wb[j]);
        for (int s0 = 0; s0 < out_steps; s0 += kMfmaDepth) {
#pragma unroll
            for (int j = 0; j < kMfmaDepth; ++j) {
                const int st = s0 + j;
                if (st < out_steps) {
                    const v8bf ca = wa[j], cb = wb[j];
                    if (st + kMfmaDepth < out_steps) load2(wr + (st + kMfmaDepth) * 64, wa[j], wb[j]);
                    v8bf ha, hbv;
                    load2(ah + st * 64, ha, hbv);
                    acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ca, ha, acc_hi, 0, 0, 0);
                    acc_lo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cb, hbv, acc_lo, 0, 0, 0);
                }
            }
        }
        if (live) {
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = rw * (acc_hi[r] + acc_lo[r]);
            atomic_add_bf16x4(quad, before, v);
        }
    }
}

unsigned grid_for(size_t items) {
    const size_t b = (items + kThreads - 1) / kThreads;
    return static_cast<unsigned>(b < 1 ? 1 : (b > 8192 ? 8192 : b));
}

}  // namespace
}  // namespace cf

using namespace cf;

extern "C" {

int cf_softmax_inplace_f32(float* d_x, int rows, int cols, cf_stream_t stream) {
    if (rows < 0 || cols < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return CF_OK;
    if (!d_x) return CF_ERR_INVALID_ARG;
    if (cols <= 64) k_softmax_wave<<<ceil_div(rows, kThreads / 64), kThreads, 0, as_stream(stream)>>>(d_x, rows, cols);
    else k_softmax_block<<<rows, kThreads, 0, as_stream(stream)>>>(d_x, cols);
    return launch_status();
}

int cf_moe_topk_route_f32(float* d_scores, int rows, int num_experts, int top_k, cf_stream_t stream,
                          float* d_row_sum_save, float* d_scores_save, int normalize_topk) {
    if (rows < 0 || num_experts < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0) return CF_OK;
    if (!d_scores) return CF_ERR_INVALID_ARG;
    if (num_experts > kMaxExpertsGeneric) return CF_ERR_UNSUPPORTED;
    hipStream_t st = as_stream(stream);
    if (num_experts <= 64) {
        k_topk_wave<true><<<ceil_div(rows, kThreads / 64), kThreads, 0, st>>>(d_scores, d_row_sum_save, d_scores_save,
                                                                               rows, num_experts, top_k, normalize_topk);
        return launch_status();
    }
    k_softmax_block<<<rows, kThreads, 0, st>>>(d_scores, num_experts);
    if (d_scores_save) {
        const hipError_t e = hipMemcpyAsync(d_scores_save, d_scores, static_cast<size_t>(rows) * num_experts * sizeof(float),
                                            hipMemcpyDeviceToDevice, st);
        if (e != hipSuccess) return static_cast<int>(e);
    }
    k_topk_wide<<<ceil_div(rows, kThreads / 64), kThreads, 0, st>>>(d_scores, d_row_sum_save, rows, num_experts, top_k, normalize_topk);
    return launch_status();
}

int cf_moe_build_expert_row_lists(const float* d_route_weights, int* d_counts, int* d_row_indices, int rows,
                                  int num_experts, cf_stream_t stream) {
    if (rows < 0 || num_experts < 0) return CF_ERR_INVALID_ARG;
    if (num_experts == 0) return CF_OK;
    if (!d_counts || (rows > 0 && (!d_route_weights || !d_row_indices))) return CF_ERR_INVALID_ARG;
    k_build_row_lists<<<num_experts, 1024, 0, as_stream(stream)>>>(d_route_weights, d_counts, d_row_indices, rows, num_experts);
    return launch_status();
}

int cf_moe_expert_offsets_from_counts(const int* d_counts, int* d_offsets, int num_experts, cf_stream_t stream) {
    if (num_experts < 0) return CF_ERR_INVALID_ARG;
    if (num_experts == 0) return CF_OK;
    if (!d_counts || !d_offsets) return CF_ERR_INVALID_ARG;
    k_offsets<<<1, 1, 0, as_stream(stream)>>>(d_counts, d_offsets, num_experts);
    return launch_status();
}

int cf_moe_gather_rows_u8(const uint8_t* d_src, uint8_t* d_dst, const int* d_row_indices, int n_rows, int width,
                          cf_stream_t stream) {
    if (n_rows < 0 || width < 0) return CF_ERR_INVALID_ARG;
    if (n_rows == 0 || width == 0) return CF_OK;
    if (!d_src || !d_dst || !d_row_indices) return CF_ERR_INVALID_ARG;
    const size_t total = static_cast<size_t>(n_rows) * width;
    if (width % 16 == 0 && aligned16(d_src) && aligned16(d_dst))
        k_gather_rows16<<<grid_for(total / 16), kThreads, 0, as_stream(stream)>>>(
            reinterpret_cast<const uint4*>(d_src), reinterpret_cast<uint4*>(d_dst), d_row_indices, n_rows, width / 16);
    else
        k_gather_rows_scalar<uint8_t><<<grid_for(total), kThreads, 0, as_stream(stream)>>>(d_src, d_dst, d_row_indices, n_rows, width);
    return launch_status();
}

int cf_moe_gather_rows_bf16(const uint16_t* d_src, uint16_t* d_dst, const int* d_row_indices, int n_rows, int width,
                            cf_stream_t stream) {
    if (n_rows < 0 || width < 0) return CF_ERR_INVALID_ARG;
    if (n_rows == 0 || width == 0) return CF_OK;
    if (!d_src || !d_dst || !d_row_indices) return CF_ERR_INVALID_ARG;
    const size_t total = static_cast<size_t>(n_rows) * width;
    if (width % 8 == 0 && aligned16(d_src) && aligned16(d_dst))
        k_gather_rows16<<<grid_for(total / 8), kThreads, 0, as_stream(stream)>>>(
            reinterpret_cast<const uint4*>(d_src), reinterpret_cast<uint4*>(d_dst), d_row_indices, n_rows, width / 8);
    else
        k_gather_rows_scalar<uint16_t><<<grid_for(total), kThreads, 0, as_stream(stream)>>>(d_src, d_dst, d_row_indices, n_rows, width);
    return launch_status();
}

int cf_moe_scatter_accumulate_rows_bf16(uint16_t* d_mixed, const uint16_t* d_compact, const float* d_route_weights,
                                        const int* d_row_indices, int n_rows, int expert_idx, int num_experts, int H,
                                        cf_stream_t stream) {
    if (n_rows < 0 || H < 0 || expert_idx < 0 || expert_idx >= num_experts) return CF_ERR_INVALID_ARG;
    if (n_rows == 0 || H == 0) return CF_OK;
    if (!d_mixed || !d_compact || !d_route_weights || !d_row_indices) return CF_ERR_INVALID_ARG;
    const int vec = H % 8 == 0 && aligned16(d_mixed) && aligned16(d_compact);
    const size_t items = static_cast<size_t>(n_rows) * (vec ? H / 8 : H);
    k_scatter_accumulate<<<grid_for(items), kThreads, 0, as_stream(stream)>>>(d_mixed, d_compact, d_route_weights, d_row_indices,
                                                                              n_rows, expert_idx, num_experts, H, vec);
    return launch_status();
}

int cf_moe_scale_accumulate_bf16(uint16_t* d_mixed, const uint16_t* d_term, const float* d_route_weights, int rows,
                                 int expert_idx, int num_experts, int H, cf_stream_t stream) {
    if (rows < 0 || H < 0 || expert_idx < 0 || expert_idx >= num_experts) return CF_ERR_INVALID_ARG;
    if (rows == 0 || H == 0) return CF_OK;
    if (!d_mixed || !d_term || !d_route_weights) return CF_ERR_INVALID_ARG;
    const int vec = H % 8 == 0 && aligned16(d_mixed) && aligned16(d_term);
    const size_t items = static_cast<size_t>(rows) * (vec ? H / 8 : H);
    k_scatter_accumulate<<<grid_for(items), kThreads, 0, as_stream(stream)>>>(d_mixed, d_term, d_route_weights, nullptr, rows,
                                                                              expert_idx, num_experts, H, vec);
    return launch_status();
}

int cf_moe_compact_row_index(const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows,
                             int num_experts, int* d_compact_index, cf_stream_t stream) {
    if (rows < 0 || num_experts < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0) return CF_OK;
    if (!d_counts || !d_offsets || !d_row_indices || !d_compact_index) return CF_ERR_INVALID_ARG;
    dim3 grid(ceil_div(rows, kThreads) < 16 ? ceil_div(rows, kThreads) : 16, num_experts);
    k_compact_index<<<grid, kThreads, 0, as_stream(stream)>>>(d_counts, d_offsets, d_row_indices, rows, d_compact_index, nullptr,
                                                              num_experts);
    return launch_status();
}

// slot_limit: the rows d_compact_out holds; (row, expert) pairs whose slot lies at or beyond it are skipped
static int unpermute_weighted(uint16_t* d_mixed, const uint16_t* d_compact_out, const float* d_route_weights,
                              const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows,
                              int num_experts, int H, int slot_limit, cf_stream_t stream) {
    if (rows < 0 || num_experts < 0 || H < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0) return CF_OK;
    if (!d_mixed || !d_compact_out || !d_route_weights || !d_counts || !d_offsets || !d_row_indices) return CF_ERR_INVALID_ARG;
    if ((H & 7) == 0 && !(aligned16(d_mixed) && aligned16(d_compact_out))) return CF_ERR_UNSUPPORTED;
    k_unpermute<false><<<rows, kThreads, 0, as_stream(stream)>>>(d_mixed, d_compact_out, d_route_weights, d_counts, d_offsets,
                                                                 d_row_indices, rows, num_experts, H, slot_limit);
    return launch_status();
}
int cf_moe_unpermute_weighted_bf16(uint16_t* d_mixed, const uint16_t* d_compact_out, const float* d_route_weights,
                                   const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows,
                                   int num_experts, int H, cf_stream_t stream) {
    return unpermute_weighted(d_mixed, d_compact_out, d_route_weights, d_counts, d_offsets, d_row_indices, rows, num_experts, H,
                              0x7fffffff, stream);
}

int cf_moe_scatter_add_rows_bf16(uint16_t* d_dst_full, const uint16_t* d_src_compact, const int* d_row_indices, int n_rows,
                                 int H, cf_stream_t stream) {
    if (n_rows < 0 || H < 0) return CF_ERR_INVALID_ARG;
    if (n_rows == 0 || H == 0) return CF_OK;
    if (!d_dst_full || !d_src_compact || !d_row_indices) return CF_ERR_INVALID_ARG;
    const int vec = H % 8 == 0 && aligned16(d_dst_full) && aligned16(d_src_compact);
    const size_t items = static_cast<size_t>(n_rows) * (vec ? H / 8 : H);
    k_scatter_accumulate<<<grid_for(items), kThreads, 0, as_stream(stream)>>>(d_dst_full, d_src_compact, nullptr, d_row_indices,
                                                                              n_rows, 0, 1, H, vec);
    return launch_status();
}

int cf_moe_unpermute_add_bf16(uint16_t* d_dst_full, const uint16_t* d_src_compact, const float* d_route_weights,
                              const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows,
                              int num_experts, int H, cf_stream_t stream) {
    if (rows < 0 || num_experts < 0 || H < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0) return CF_OK;
    if (!d_dst_full || !d_src_compact || !d_route_weights || !d_counts || !d_offsets || !d_row_indices) return CF_ERR_INVALID_ARG;
    if ((H & 7) == 0 && !(aligned16(d_dst_full) && aligned16(d_src_compact))) return CF_ERR_UNSUPPORTED;
    k_unpermute<true><<<rows, kThreads, 0, as_stream(stream)>>>(d_dst_full, d_src_compact, d_route_weights, d_counts, d_offsets,
                                                                d_row_indices, rows, num_experts, H, 0x7fffffff);
    return launch_status();
}

int cf_moe_build_slot_index(const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows, int num_experts,
                            int* d_slot_index, cf_stream_t stream) {
    if (rows < 0 || num_experts < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0) return CF_OK;
    if (!d_counts || !d_offsets || !d_row_indices || !d_slot_index) return CF_ERR_INVALID_ARG;
    const dim3 grid(ceil_div(static_cast<size_t>(rows), kThreads * 4), num_experts);
    k_slot_index<<<grid, kThreads, 0, as_stream(stream)>>>(d_counts, d_offsets, d_row_indices, rows, num_experts, d_slot_index);
    return launch_status();
}

static int unpermute_indexed(uint16_t* d_mixed, const uint16_t* d_compact_out, const float* d_route_weights,
                             const int* d_slot_index, int rows, int num_experts, int H, int unit_weights, int slot_limit,
                             cf_stream_t stream) {
    if (rows < 0 || num_experts < 0 || H < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0) return CF_OK;
    if (!d_mixed || !d_compact_out || !d_route_weights || !d_slot_index) return CF_ERR_INVALID_ARG;
    if ((H & 7) == 0 && !(aligned16(d_mixed) && aligned16(d_compact_out))) return CF_ERR_UNSUPPORTED;
    if (unit_weights)
        k_unpermute_indexed<true><<<rows, kThreads, 0, as_stream(stream)>>>(d_mixed, d_compact_out, d_route_weights, d_slot_index,
                                                                            num_experts, H, slot_limit);
    else
        k_unpermute_indexed<false><<<rows, kThreads, 0, as_stream(stream)>>>(d_mixed, d_compact_out, d_route_weights, d_slot_index,
                                                                             num_experts, H, slot_limit);
    return launch_status();
}
int cf_moe_unpermute_indexed_bf16(uint16_t* d_mixed, const uint16_t* d_compact_out, const float* d_route_weights,
                                  const int* d_slot_index, int rows, int num_experts, int H, int unit_weights,
                                  cf_stream_t stream) {
    return unpermute_indexed(d_mixed, d_compact_out, d_route_weights, d_slot_index, rows, num_experts, H, unit_weights, 0x7fffffff,
                             stream);
}

// ---- grouped SwiGLU expert bank -----------------------------------------------------------------
namespace {
struct SwigluWs { size_t tile_map, index, act, actq, act_scale, act_descale, y, slot, slot_bytes, total; };
SwigluWs swiglu_layout(int total_rows, int num_experts, int H, int Ie) {
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    SwigluWs w{};
    size_t map_bytes = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_rows, num_experts, &map_bytes);
    size_t off = 0;
    w.tile_map = off; off = up(off + map_bytes);
    w.index = off; off = up(off + sizeof(int) * static_cast<size_t>(total_rows));
    w.act = off; off = up(off + 2 * static_cast<size_t>(total_rows) * Ie);
    w.actq = off; off = up(off + static_cast<size_t>(total_rows) * Ie);
    w.act_scale = off; off = up(off + sizeof(float) * static_cast<size_t>(total_rows));
    w.act_descale = off; off = up(off + sizeof(float) * static_cast<size_t>(total_rows));
    w.y = off; off = up(off + 2 * static_cast<size_t>(total_rows) * H);
    // the (row, expert) -> slot table of the unpermute: rows <= total_rows whenever every row selects an expert;
    // a caller with more rows than that, or a table beyond 64 MiB, gets the searching unpermute instead
    w.slot_bytes = sizeof(int) * static_cast<size_t>(total_rows) * num_experts;
    if (w.slot_bytes > (64u << 20)) w.slot_bytes = 0;
    w.slot = off; off = up(off + w.slot_bytes);
    w.total = off;
    return w;
}
}  // namespace

int cf_moe_grouped_swiglu_workspace_bytes(int total_selected_rows, int num_experts, int H, int Ie, size_t* bytes) {
    if (total_selected_rows < 0 || num_experts < 0 || H < 0 || Ie < 0 || !bytes) return CF_ERR_INVALID_ARG;
    *bytes = swiglu_layout(total_selected_rows, num_experts, H, Ie).total;
    return CF_OK;
}

int cf_moe_grouped_swiglu_forward_fp8(const void* d_hidden_e4m3, const float* d_hidden_descale,
                                      const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                      const int* d_row_indices, const void* d_w_gate, const float* d_w_gate_descale,
                                      const void* d_w_up, const float* d_w_up_descale, const void* d_w_down,
                                      const float* d_w_down_descale, uint16_t* d_mixed, int rows, int H, int Ie,
                                      int num_experts, int total_selected_rows, void* d_workspace,
                                      size_t workspace_bytes, cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0 || total_selected_rows < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || total_selected_rows == 0) return CF_OK;
    if (!d_hidden_e4m3 || !d_hidden_descale || !d_route_weights || !d_counts || !d_offsets || !d_row_indices ||
        !d_w_gate || !d_w_gate_descale || !d_w_up || !d_w_up_descale || !d_w_down || !d_w_down_descale || !d_mixed ||
        !d_workspace)
        return CF_ERR_INVALID_ARG;
    const SwigluWs w = swiglu_layout(total_selected_rows, num_experts, H, Ie);
    if (workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(d_workspace) & 255u)) return CF_ERR_INVALID_ARG;
    auto* base = static_cast<uint8_t*>(d_workspace);
    int* index = reinterpret_cast<int*>(base + w.index);
    auto* act = reinterpret_cast<uint16_t*>(base + w.act);
    auto* actq = base + w.actq;
    auto* act_scale = reinterpret_cast<float*>(base + w.act_scale);
    auto* act_descale = reinterpret_cast<float*>(base + w.act_descale);
    auto* y = reinterpret_cast<uint16_t*>(base + w.y);
    size_t map_bytes = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_selected_rows, num_experts, &map_bytes);
    // the compact index for the gather and, when the workspace holds it, its inverse for the unpermute: one launch
    const bool indexed = sizeof(int) * static_cast<size_t>(rows) * num_experts <= w.slot_bytes;
    int* slot = indexed ? reinterpret_cast<int*>(base + w.slot) : nullptr;
    // with the tile table of both projections in the same launch
    bank_setup(d_counts, d_row_indices, rows, num_experts, total_selected_rows, nullptr, index, slot,
               reinterpret_cast<int*>(base + w.tile_map), as_stream(stream));
    int rc = launch_status();
    if (rc) return rc;
    // gate/up: rows gathered through the compact index (the token permute is fused into the operand fetch)
    rc = grouped_gemm_nt_bf16(total_selected_rows, Ie, H, num_experts, d_counts, d_offsets, d_hidden_e4m3, rows, H, index,
                              d_hidden_descale, d_w_gate, d_w_gate_descale, CF_SCALE_ROW_COL, CF_EPI_SILU_GATE, d_w_up, d_w_up_descale,
                              act, Ie, base + w.tile_map, map_bytes, false, 0, stream);
    if (rc) return rc;
    rc = cf_fp8_quantize_rows(act, total_selected_rows, Ie, 0, actq, act_scale, act_descale, stream);
    if (rc) return rc;
    // same routing, same tile table
    rc = grouped_gemm_nt_bf16(total_selected_rows, H, Ie, num_experts, d_counts, d_offsets, actq, total_selected_rows, Ie, nullptr,
                              act_descale, d_w_down, d_w_down_descale, CF_SCALE_ROW_COL, CF_EPI_NONE, nullptr, nullptr, y, H,
                              base + w.tile_map, map_bytes, false, 0, stream);
    if (rc) return rc;
    if (indexed) return unpermute_indexed(d_mixed, y, d_route_weights, slot, rows, num_experts, H, 0, total_selected_rows, stream);
    return unpermute_weighted(d_mixed, y, d_route_weights, d_counts, d_offsets, d_row_indices, rows, num_experts, H,
                              total_selected_rows, stream);
}

// ---- grouped GELU expert bank on the matrix cores -----------------------------------------------
// The reference's per-expert loop (gather -> FP8 GEMM -> gelu_forward -> quantize -> FP8 GEMM -> scatter-accumulate,
// src/trainer.cu:6886-6934) for all experts at once.  The workspace is the SwiGLU bank's plus the three per-tensor
// descales spread into the per-token / per-channel vectors the grouped GEMM reads.
namespace {
struct GeluWs { SwigluWs s; size_t hidden_descale, in_descale, out_descale, total; };
GeluWs gelu_layout(int rows, int total_rows, int num_experts, int H, int Ie) {
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    GeluWs w{};
    w.s = swiglu_layout(total_rows, num_experts, H, Ie);
    size_t off = w.s.total;
    w.hidden_descale = off; off = up(off + sizeof(float) * static_cast<size_t>(rows));
    w.in_descale = off; off = up(off + sizeof(float) * static_cast<size_t>(num_experts) * Ie);
    w.out_descale = off; off = up(off + sizeof(float) * static_cast<size_t>(num_experts) * H);
    w.total = off;
    return w;
}

__global__ __launch_bounds__(kThreads) void k_spread_descales(const float* __restrict__ a, float* __restrict__ av, size_t na,
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
}  // namespace

int cf_moe_grouped_gelu_workspace_bytes(int rows, int total_selected_rows, int num_experts, int H, int Ie, size_t* bytes) {
    if (rows < 0 || total_selected_rows < 0 || num_experts < 0 || H < 0 || Ie < 0 || !bytes) return CF_ERR_INVALID_ARG;
    *bytes = gelu_layout(rows, total_selected_rows, num_experts, H, Ie).total;
    return CF_OK;
}

namespace {
// The per-expert activation slots of the loop's fc_out input (moe_fcout_act_slot, src/trainer.cu:6916): null states =
// one scale per token row instead.
struct FcoutSlots { float* states; int stride, history_len, is_e5m2, is_recompute; };

int gelu_bank_forward(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                      const float* d_route_weights, const int* d_counts, const int* d_offsets,
                      const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                      const void* d_fc_out_w, const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                      int H, int Ie, int num_experts, int total_selected_rows, const FcoutSlots& slots, void* d_workspace,
                      size_t workspace_bytes, cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0 || total_selected_rows < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || total_selected_rows == 0) return CF_OK;
    if (!d_hidden || !d_fcin_descale || !d_route_weights || !d_counts || !d_offsets || !d_row_indices || !d_fc_in_w ||
        !d_fc_in_descale || !d_fc_out_w || !d_fc_out_descale || !d_mixed || !d_workspace)
        return CF_ERR_INVALID_ARG;
    const GeluWs w = gelu_layout(rows, total_selected_rows, num_experts, H, Ie);
    if (workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(d_workspace) & 255u)) return CF_ERR_INVALID_ARG;
    auto* base = static_cast<uint8_t*>(d_workspace);
    int* index = reinterpret_cast<int*>(base + w.s.index);
    auto* act = reinterpret_cast<uint16_t*>(base + w.s.act);
    auto* actq = base + w.s.actq;
    auto* act_scale = reinterpret_cast<float*>(base + w.s.act_scale);
    auto* act_descale = reinterpret_cast<float*>(base + w.s.act_descale);
    auto* y = reinterpret_cast<uint16_t*>(base + w.s.y);
    auto* hidden_descale = reinterpret_cast<float*>(base + w.hidden_descale);
    auto* in_descale = reinterpret_cast<float*>(base + w.in_descale);
    auto* out_descale = reinterpret_cast<float*>(base + w.out_descale);
    size_t map_bytes = 0;
    cf_fp8_grouped_gemm_workspace_bytes(total_selected_rows, num_experts, &map_bytes);
    hipStream_t st = as_stream(stream);
    const bool indexed = sizeof(int) * static_cast<size_t>(rows) * num_experts <= w.s.slot_bytes;
    int* slot = indexed ? reinterpret_cast<int*>(base + w.s.slot) : nullptr;
    bank_setup(d_counts, d_row_indices, rows, num_experts, total_selected_rows, nullptr, index, slot,
               reinterpret_cast<int*>(base + w.s.tile_map), st);
    int rc = launch_status();
    if (rc) return rc;
    {
        const size_t na = static_cast<size_t>(rows), nb = static_cast<size_t>(num_experts) * Ie, nc = static_cast<size_t>(num_experts) * H;
        k_spread_descales<<<grid_for(na + nb + nc), kThreads, 0, st>>>(d_fcin_descale, hidden_descale, na, d_fc_in_descale, in_descale, nb,
                                                                      d_fc_out_descale, out_descale, nc);
    }
    rc = launch_status();
    if (rc) return rc;
    // fc_in: token rows gathered through the compact index in the operand fetch
    rc = grouped_gemm_nt_bf16(total_selected_rows, Ie, H, num_experts, d_counts, d_offsets, d_hidden, rows, H, index, hidden_descale,
                              d_fc_in_w, in_descale, CF_SCALE_ROW_COL, CF_EPI_NONE, nullptr, nullptr, act, Ie, base + w.s.tile_map,
                              map_bytes, false, fcin_is_e5m2 ? 1 : 0, stream);
    if (rc) return rc;
    // gelu_forward and the quantize in one pass over the bf16 projections: one scale per token row, or the loop's own
    // per-expert delayed scale (fp8_quant_act on the expert's slot, src/trainer.cu:6916-6918), whose snapshot descale
    // is spread over the expert's rows for the GEMM
    if (slots.states)
        rc = cf_moe_grouped_quantize_delayed(act, actq, Ie, num_experts, d_counts, d_offsets, total_selected_rows, slots.states,
                                             slots.stride, slots.history_len, slots.is_e5m2, 1, slots.is_recompute, act_descale, stream);
    else
        rc = cf_gelu_quantize_rows_e4m3(act, total_selected_rows, Ie, actq, act_scale, act_descale, stream);
    if (rc) return rc;
    rc = grouped_gemm_nt_bf16(total_selected_rows, H, Ie, num_experts, d_counts, d_offsets, actq, total_selected_rows, Ie, nullptr,
                              act_descale, d_fc_out_w, out_descale, CF_SCALE_ROW_COL, CF_EPI_NONE, nullptr, nullptr, y, H,
                              base + w.s.tile_map, map_bytes, false, slots.states && slots.is_e5m2 ? 1 : 0, stream);
    if (rc) return rc;
    if (indexed) return unpermute_indexed(d_mixed, y, d_route_weights, slot, rows, num_experts, H, 0, total_selected_rows, stream);
    return unpermute_weighted(d_mixed, y, d_route_weights, d_counts, d_offsets, d_row_indices, rows, num_experts, H,
                              total_selected_rows, stream);
}
}  // namespace

int cf_moe_grouped_gelu_forward_fp8(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                    const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                    const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                    const void* d_fc_out_w, const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                    int H, int Ie, int num_experts, int total_selected_rows, void* d_workspace,
                                    size_t workspace_bytes, cf_stream_t stream) {
    return gelu_bank_forward(d_hidden, d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts, d_offsets, d_row_indices, d_fc_in_w,
                             d_fc_in_descale, d_fc_out_w, d_fc_out_descale, d_mixed, rows, H, Ie, num_experts, total_selected_rows,
                             FcoutSlots{nullptr, 0, 0, 0, 0}, d_workspace, workspace_bytes, stream);
}

int cf_moe_grouped_gelu_forward_fp8_slots(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                          const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                          const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                          const void* d_fc_out_w, const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                          int H, int Ie, int num_experts, int total_selected_rows, float* d_fcout_slot_states,
                                          int state_stride_words, int history_len, int fcout_is_e5m2, int is_recompute,
                                          void* d_workspace, size_t workspace_bytes, cf_stream_t stream) {
    if (!d_fcout_slot_states || history_len < 0 || state_stride_words < cf_act_slot_state_words(history_len)) return CF_ERR_INVALID_ARG;
    return gelu_bank_forward(d_hidden, d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts, d_offsets, d_row_indices, d_fc_in_w,
                             d_fc_in_descale, d_fc_out_w, d_fc_out_descale, d_mixed, rows, H, Ie, num_experts, total_selected_rows,
                             FcoutSlots{d_fcout_slot_states, state_stride_words, history_len, fcout_is_e5m2 ? 1 : 0, is_recompute ? 1 : 0},
                             d_workspace, workspace_bytes, stream);
}

int cf_moe_grouped_expert_forward_fp8(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                      const float* d_route_weights, const int* d_counts, const int* d_offsets,
                                      const int* d_row_indices, const void* d_fc_in_w, const float* d_fc_in_descale,
                                      const void* d_fc_out_w, const float* d_fc_out_descale, uint16_t* d_mixed, int rows,
                                      int H, int Ie, int num_experts, int total_selected_rows, cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0 || Ie == 0) return CF_OK;
    if (!d_hidden || !d_fcin_descale || !d_route_weights || !d_counts || !d_row_indices || !d_fc_in_w || !d_fc_in_descale ||
        !d_fc_out_w || !d_fc_out_descale || !d_mixed)
        return CF_ERR_INVALID_ARG;
    (void)d_offsets;               // accepted and unused, as in the reference (kernels/moe.cu:1063-1071)
    (void)total_selected_rows;
    return expert_forward_fp8_one_kernel(d_hidden, d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts, d_row_indices, d_fc_in_w,
                                         d_fc_in_descale, d_fc_out_w, d_fc_out_descale, d_mixed, rows, H, Ie, num_experts, stream);
}

}  // extern "C"

int cf::expert_forward_fp8_one_kernel(const void* d_hidden, const float* d_fcin_descale, int fcin_is_e5m2,
                                      const float* d_route_weights, const int* d_counts, const int* d_row_indices,
                                      const void* d_fc_in_w, const float* d_fc_in_descale, const void* d_fc_out_w,
                                      const float* d_fc_out_descale, uint16_t* d_mixed, int rows, int H, int Ie, int num_experts,
                                      cf_stream_t stream) {
    const bool mfma_ok = H % 128 == 0 && Ie % 64 == 0 && aligned16(d_hidden) && aligned16(d_fc_in_w) && aligned16(d_fc_out_w) &&
                         (reinterpret_cast<uintptr_t>(d_mixed) & 7u) == 0;
    // 32 rows per workgroup where the output blocks fit a wavefront's registers and LDS holds the hidden rows plus
    // a chunk of at least 64 activation columns: Ie is walked in the fewest equal chunks that fit
    if (mfma_ok && H <= 128 * kWideBlocks) {
        const long long room = 160 * 1024 - static_cast<long long>(kWideRows) * (H + 16);
        const int max_chunk = room > 0 ? static_cast<int>(((room / (4 * kWideRows)) - 8) / 64 * 64) : 0;
        if (max_chunk >= 64) {
            const int passes = (Ie + max_chunk - 1) / max_chunk;
            const int chunk = ((Ie + passes - 1) / passes + 63) / 64 * 64;
            const size_t smem32 = static_cast<size_t>(kWideRows) * (H + 16) + 4u * kWideRows * (static_cast<size_t>(chunk) + 8);
            static std::once_flag once32;
            static hipError_t err32 = hipSuccess;
            std::call_once(once32, [] {
                err32 = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_grouped_gelu_fp8_mfma32<false>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (err32 == hipSuccess)
                    err32 = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_grouped_gelu_fp8_mfma32<true>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            });
            if (err32 != hipSuccess) return static_cast<int>(err32);
            const int tiles = (rows + kWideRows - 1) / kWideRows;
            auto launch = [&](auto kernel) {
                kernel<<<kXcdCount * ((num_experts + kXcdCount - 1) / kXcdCount) * tiles, kMfmaThreads, smem32, as_stream(stream)>>>(
                    static_cast<const uint8_t*>(d_hidden), d_fcin_descale, d_route_weights, d_counts, d_row_indices,
                    static_cast<const uint8_t*>(d_fc_in_w), d_fc_in_descale, static_cast<const uint8_t*>(d_fc_out_w), d_fc_out_descale,
                    d_mixed, rows, H, Ie, num_experts, tiles, chunk);
            };
            if (fcin_is_e5m2) launch(k_grouped_gelu_fp8_mfma32<true>);
            else launch(k_grouped_gelu_fp8_mfma32<false>);
            return launch_status();
        }
    }
    // the matrix-core form where the shapes are whole MFMA steps and its tile fits the LDS
    const size_t smem_mfma = static_cast<size_t>(kMfmaRows) * (H + 16) + 4u * kMfmaRows * (static_cast<size_t>(Ie) + 8);
    if (H % 128 == 0 && Ie % 64 == 0 && smem_mfma <= 160 * 1024 && aligned16(d_hidden) && aligned16(d_fc_in_w) &&
        aligned16(d_fc_out_w) && (reinterpret_cast<uintptr_t>(d_mixed) & 7u) == 0) {
        static std::once_flag once_mfma;
        static hipError_t err_mfma = hipSuccess;
        std::call_once(once_mfma, [] {
            err_mfma = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_grouped_gelu_fp8_mfma<false>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (err_mfma == hipSuccess)
                err_mfma = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_grouped_gelu_fp8_mfma<true>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        });
        if (err_mfma != hipSuccess) return static_cast<int>(err_mfma);
        const int tiles = (rows + kMfmaRows - 1) / kMfmaRows;
        auto launch = [&](auto kernel) {
            kernel<<<kXcdCount * ((num_experts + kXcdCount - 1) / kXcdCount) * tiles, kMfmaThreads, smem_mfma, as_stream(stream)>>>(
                static_cast<const uint8_t*>(d_hidden), d_fcin_descale, d_route_weights, d_counts, d_row_indices,
                static_cast<const uint8_t*>(d_fc_in_w), d_fc_in_descale, static_cast<const uint8_t*>(d_fc_out_w), d_fc_out_descale,
                d_mixed, rows, H, Ie, num_experts, tiles);
        };
        if (fcin_is_e5m2) launch(k_grouped_gelu_fp8_mfma<true>);
        else launch(k_grouped_gelu_fp8_mfma<false>);
        return launch_status();
    }
    return launch_grouped_gelu_wave<false>(static_cast<const uint8_t*>(d_hidden), d_fcin_descale, fcin_is_e5m2, d_route_weights, d_counts,
                                           d_row_indices, static_cast<const uint8_t*>(d_fc_in_w), d_fc_in_descale,
                                           static_cast<const uint8_t*>(d_fc_out_w), d_fc_out_descale, d_mixed, rows, H, Ie, num_experts,
                                           as_stream(stream));
}

extern "C" {

int cf_moe_grouped_expert_forward_bf16(const uint16_t* d_hidden, const float* d_route_weights, const int* d_counts,
                                       const int* d_offsets, const int* d_row_indices, const uint16_t* d_fc_in_w,
                                       const uint16_t* d_fc_out_w, uint16_t* d_mixed, int rows, int H, int Ie,
                                       int num_experts, int total_selected_rows, cf_stream_t stream) {
    if (rows < 0 || H < 0 || Ie < 0 || num_experts < 0) return CF_ERR_INVALID_ARG;
    if (rows == 0 || num_experts == 0 || H == 0 || Ie == 0) return CF_OK;
    if (!d_hidden || !d_route_weights || !d_counts || !d_row_indices || !d_fc_in_w || !d_fc_out_w || !d_mixed) return CF_ERR_INVALID_ARG;
    (void)d_offsets;               // the row lists carry everything the kernels need
    (void)total_selected_rows;     // the reference's launch bound (kernels/moe.cu:875); the grid here follows the row lists
    return expert_forward_bf16_one_kernel(d_hidden, d_route_weights, d_counts, d_row_indices, d_fc_in_w, d_fc_out_w, d_mixed, rows, H, Ie,
                                          num_experts, stream);
}

}  // extern "C"

int cf::expert_forward_bf16_one_kernel(const uint16_t* d_hidden, const float* d_route_weights, const int* d_counts,
                                       const int* d_row_indices, const uint16_t* d_fc_in_w, const uint16_t* d_fc_out_w,
                                       uint16_t* d_mixed, int rows, int H, int Ie, int num_experts, cf_stream_t stream) {
    // the matrix-core form where the shapes are whole MFMA steps and its tile fits the LDS
    const size_t smem_mfma = 2u * kMfmaRows * (static_cast<size_t>(H) + 8) + 2u * kMfmaRows * (static_cast<size_t>(Ie) + 8);
    if (H % 64 == 0 && Ie % 64 == 0 && smem_mfma <= 160 * 1024 && aligned16(d_hidden) && aligned16(d_fc_in_w) && aligned16(d_fc_out_w) &&
        (reinterpret_cast<uintptr_t>(d_mixed) & 7u) == 0) {
        static std::once_flag once_mfma;
        static hipError_t err_mfma = hipSuccess;
        std::call_once(once_mfma, [] {
            err_mfma = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_grouped_gelu_bf16_mfma),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        });
        if (err_mfma != hipSuccess) return static_cast<int>(err_mfma);
        const int tiles = (rows + kMfmaRows - 1) / kMfmaRows;
        k_grouped_gelu_bf16_mfma<<<kXcdCount * ((num_experts + kXcdCount - 1) / kXcdCount) * tiles, kMfmaThreads, smem_mfma, as_stream(stream)>>>(
            d_hidden, d_route_weights, d_counts, d_row_indices, d_fc_in_w, d_fc_out_w, d_mixed, rows, H, Ie, num_experts, tiles);
        return launch_status();
    }
    return launch_grouped_gelu_wave<true>(reinterpret_cast<const uint8_t*>(d_hidden), nullptr, 0, d_route_weights, d_counts, d_row_indices,
                                          reinterpret_cast<const uint8_t*>(d_fc_in_w), nullptr, reinterpret_cast<const uint8_t*>(d_fc_out_w),
                                          nullptr, d_mixed, rows, H, Ie, num_experts, as_stream(stream));
}

// mixed[row] += w[row, e] * y[slot(row, e)] over the row's experts in ascending order for fp32 rows of y, one bf16
// rounding per expert; the slot table when the caller has one, the search of the row lists otherwise
int cf::unpermute_f32(uint16_t* d_mixed, const float* d_y, const float* d_route_weights, const int* d_slot_index,
                      const int* d_counts, const int* d_offsets, const int* d_row_indices, int rows, int num_experts, int H,
                      int slot_limit, hipStream_t st) {
    if (rows <= 0 || num_experts <= 0 || H <= 0) return CF_OK;
    if ((H & 7) == 0 && !(aligned16(d_mixed) && aligned16(d_y))) return CF_ERR_UNSUPPORTED;
    if (d_slot_index)
        k_unpermute_indexed<false, float><<<rows, kThreads, 0, st>>>(d_mixed, d_y, d_route_weights, d_slot_index, num_experts, H, slot_limit);
    else
        k_unpermute<false, float><<<rows, kThreads, 0, st>>>(d_mixed, d_y, d_route_weights, d_counts, d_offsets, d_row_indices, rows,
                                                            num_experts, H, slot_limit);
    return launch_status();
}
