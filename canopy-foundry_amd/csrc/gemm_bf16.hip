// bf16 GEMMs of the selected-expert MoE backward, dense and grouped per expert.
//
// The reference runs four cuBLAS calls per expert behind a host copy of the counts (src/trainer.cu:7727-7740,
// wrappers :3069-3160): two input gradients  C[n,N] = A[n,K] . B[K,N]  (gemm_bf16, row-major, beta = 0) and two
// weight gradients  C[M,N] += A[n,M]^T . B[n,N]  (gemm_bf16_tn_f32, beta = 1, the contraction runs over the
// expert's n rows).  Here one launch covers every expert, with the counts and offsets read on the device.
//
// In both forms at least one operand is stored with the contraction index as its SLOW dimension, while an MFMA
// lane needs eight consecutive k of one row (or column).  Such a tile is parked in LDS as it lies in memory,
// [k][columns], and read with ds_read_b64_tr_b16: per 16 lanes the instruction takes a 4 (k) x 16 (columns) block,
// source lane r supplying the address of row r / 4, columns 4 (r % 4) .. +3, and hands lane i the four k values of
// column i.  Two such reads give a lane its eight k of a 32x32x16 MFMA operand.  An operand that is K-contiguous
// in memory takes the usual path (128-byte LDS rows, 16-byte chunks xor-swizzled, ds_read_b128).
//
// Workgroup tile 256 (M) x 256 (N) x 64 (K), four wavefronts 2 x 2, each 128 x 128 = 4 x 4 tiles of
// v_mfma_f32_32x32x16_bf16 with fp32 accumulators.  The N-side operand goes to the MFMA "A" side, so a lane
// ends up with four consecutive output columns of one output row per accumulator quad.  Global loads are
// register staged two K-tiles ahead (16 bytes per lane), LDS is double buffered, one barrier per K-tile.
// Rows, columns and k beyond the operands' bounds are read as zeros (buffer loads with the operand's size in their
// descriptor), so any n_e works.
#include "common.hpp"
#include "internal.hpp"

#include <mutex>
#include <type_traits>

namespace cf {
namespace {

constexpr int TM = 256, TN = 256, kThr = 256;
constexpr int kMaxTK = 64;
constexpr int kPitchKC = kMaxTK * 2;           // a K-contiguous tile: 128-byte rows, chunks swizzled
constexpr int kPitchM = TM * 2 + 64;           // a [k][m] tile of the M side: 576-byte rows
constexpr int kPitchN = TN * 2 + 64;           // a [k][n] tile of the N side: 576-byte rows
// the pads put four consecutive k rows into four different quarters of the 256 bytes the banks span
constexpr int kATile = kMaxTK * kPitchM;           // 36,864 bytes: covers both forms of the M-side tile (K-contiguous: 32,768)
constexpr int kBTile = kMaxTK * kPitchN;           // 36,864 bytes
constexpr int kStage = kATile + kBTile;
constexpr int kLds = 2 * kStage;               // 147,456 bytes: one workgroup per CU

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4bf* lds_v4bf_ptr;

enum { OUT_STORE_BF16 = 0, OUT_ACCUM_BF16 = 1, OUT_ACCUM_F32 = 2, OUT_STORE_F32 = 3 };

struct BfArgs {
    const uint16_t* A; int lda;     // M side.  NN: [M rows][K]; TN: [K rows][M]
    const uint16_t* B; int ldb;     // N side: [K rows][N]; NT (B_KC): [N rows][K]
    void* C; int ldc;               // [M][N], bf16 or fp32
    int M, N, K;
    int tiles_m, tiles_n;
    int num_experts;
    // grouped forms
    const int* counts; const int* offsets;
    const int* tile_map;            // NN: [0] = row tiles, then (expert, first row, end row, first row tile, row tiles) each
    long long b_expert_stride;      // NN: elements between the experts' B matrices
    long long c_expert_stride;      // TN: elements between the experts' C matrices
    const int* a_row_index;         // NT, GATHER: row r of the M side is row a_row_index[r] of A (a_rows rows in all)
    int a_rows;
    int b_k_period;                 // NT: B has this many columns and k runs over them again and again (K a multiple:
                                    // A's rows are several terms side by side against the same B); 0 = B has K columns
};

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// An accumulator element as a vector-ALU operand.  The explicit read keeps the register allocator from moving whole
// accumulator tiles into ordinary registers around the epilogue.
__device__ __forceinline__ float acc_read(float a) {
    float v;
    asm("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}

__device__ __forceinline__ int swz(int row) { return (row ^ ((row >> 3) & 3)) & 7; }

// Eight k of one column for every lane: two transposing reads of a [k][columns] tile.  `lane_ptr` is the tile's base
// plus this lane's share of the address (ks_lane_offset); the k-step and the column block are compile-time
// constants, so they end up in the instructions' immediate offsets and no address register is spent on them.
__device__ __forceinline__ int ks_lane_offset(int pitch, int lane) {
    const int b = lane >> 4, r = lane & 15;
    return (8 * (b >> 1) + (r >> 2)) * pitch + (16 * (b & 1) + 4 * (r & 3)) * 2;
}
template <int PITCH>
__device__ __forceinline__ v8bf read_ks(const uint8_t* lane_ptr, int krow0, int col0) {
    const uint8_t* p = lane_ptr + krow0 * PITCH + col0 * 2;
    const v4bf lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4bf_ptr)(p));
    const v4bf hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4bf_ptr)(p + 4 * PITCH));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// A_KS: the M-side operand is stored [K][M] (the weight-gradient form); otherwise [M][K].
// B_KC: the N-side operand is stored [N][K] (a weight matrix as the forward pass holds it); otherwise [K][N].
// GATHER (with the [M][K] form of A): the tile's rows of A are fetched through a row index, so a token permute
// needs no pass of its own.
template <bool A_KS, int OUT, bool GROUPED, bool B_KC = false, bool GATHER = false>
__global__ __launch_bounds__(kThr) __attribute__((amdgpu_waves_per_eu(1, 1)))
void k_gemm_bf16(const BfArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- which tile ----
    // Workgroups go to the 8 XCDs round-robin (launch position % 8), each XCD with its own 4 MiB L2.  Position b is
    // therefore read as (XCD x = b % 8, that XCD's i-th workgroup), and what an XCD runs at one time is made to share
    // operands: in the row-major forms XCD x walks the contiguous range [x * per, (x + 1) * per) of the tile order in
    // patches of 8 row tiles x 4 column tiles; in the grouped weight-gradient form XCD x owns experts x, x + 8, ...
    // whole, so that all tiles of an expert stream the same rows through one L2.
    const int x = blockIdx.x % 8, xi = blockIdx.x / 8;
    int m0, n0, m_end = p.M, k_begin = 0, k_end = p.K;
    const uint16_t* B = p.B;
    size_t c_base = 0;
    if constexpr (GROUPED && A_KS) {
        const int tiles = p.tiles_m * p.tiles_n;
        const int e = x + 8 * (xi / tiles), t = xi % tiles;
        if (e >= p.num_experts) return;
        m0 = (t % p.tiles_m) * TM;
        n0 = (t / p.tiles_m) * TN;
        // uniform values, but loaded through the vector path: moved to scalar registers, where the descriptors need them
        k_begin = __builtin_amdgcn_readfirstlane(p.offsets[e]);
        k_end = k_begin + __builtin_amdgcn_readfirstlane(p.counts[e]);
        c_base = static_cast<size_t>(e) * p.c_expert_stride;
    } else {
        const int row_tiles = GROUPED ? __builtin_amdgcn_readfirstlane(p.tile_map[0]) : p.tiles_m;
        const int total = row_tiles * p.tiles_n;
        const int per = (total + 7) / 8;
        const int t = x * per + xi;
        if (xi >= per || t >= total) return;
        constexpr int GM = 8;
        const int group = t / (GM * p.tiles_n), first = group * GM;
        const int gm = min(GM, row_tiles - first), in_group = t - group * GM * p.tiles_n;
        const int tmi = first + in_group % gm;
        n0 = (in_group / gm) * TN;
        m0 = tmi * TM;
        if constexpr (GROUPED) {
            const int* e = p.tile_map + 1 + 5 * tmi;
            const int expert = __builtin_amdgcn_readfirstlane(e[0]), first_row = __builtin_amdgcn_readfirstlane(e[1]);
            const int end_row = __builtin_amdgcn_readfirstlane(e[2]), first_tile = __builtin_amdgcn_readfirstlane(e[3]);
            m0 = first_row + (tmi - first_tile) * TM;
            m_end = min(m0 + TM, end_row);
            B += static_cast<size_t>(expert) * p.b_expert_stride;
        }
    }
    if (k_end <= k_begin) {
        if constexpr (OUT == OUT_ACCUM_BF16 || OUT == OUT_ACCUM_F32) return;      // nothing to add
    }
    constexpr int TK = 64;
    constexpr int NA = A_KS ? TK / 8 : 8, NB = TK / 8;       // 16-byte chunks per lane and K-tile
    const int nk = (k_end - k_begin + TK - 1) / TK;

    // ---- global -> registers -> LDS: 16-byte chunks through buffer loads ----
    // A buffer load takes a descriptor with a base and a size in bytes and returns zeros for a lane whose offset lies
    // beyond the size, so every load is issued unconditionally (loads under branches would keep the compiler from
    // counting the loads in flight: it would wait for all of them, the prefetch included, before the first LDS store)
    // and the zero fill of the ragged ends costs nothing.  Each load gets a descriptor of its own, built with scalar
    // instructions: the base is the first of the eight-row (32-row) group it fetches, the size what is left of the
    // operand from there (nothing, past the end of the k range), so the lane's offset is one constant per operand: its
    // row within the group and its 16-byte column; a lane whose columns lie outside the operand (or, for the
    // K-contiguous form, whose k chunk lies beyond K) uses an offset beyond every size.  The launcher keeps operands
    // below 2 GiB.
    constexpr uint32_t kOutside = 0x80000000u;
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    // rows [row0, row_end) of a row-major operand with `ld` elements per row, seen from element `col0` of row row0
    auto load_rows = [](const uint16_t* base, int ld, int row0, int row_end, int col0, uint32_t lane_off) {
        const int rows_left = max(row_end - row0, 0);
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(base + static_cast<size_t>(row0) * ld + col0), 0,
            static_cast<int>(static_cast<uint32_t>(rows_left) * static_cast<uint32_t>(ld) * 2u), 0x00020000);
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<int>(lane_off), 0, 0);
        return make_uint4(v.x, v.y, v.z, v.w);
    };
    // [k][columns] operands: this lane's row within a group of eight k rows and its 16-byte column
    const uint32_t b_lane = n0 + (tid & 31) * 8 < p.N ? (tid >> 5) * static_cast<uint32_t>(p.ldb) * 2u + (tid & 31) * 16u : kOutside;
    const uint32_t a_lane_ks = m0 + (tid & 31) * 8 < p.M ? (tid >> 5) * static_cast<uint32_t>(p.lda) * 2u + (tid & 31) * 16u : kOutside;
    // [m][k] operand: this lane's row within a group of 32 rows and its 16-byte k chunk
    const uint32_t a_lane_kc = (tid >> 3) * static_cast<uint32_t>(p.lda) * 2u + (tid & 7) * 16u;
    const uint32_t b_lane_kc = (tid >> 3) * static_cast<uint32_t>(p.ldb) * 2u + (tid & 7) * 16u;
    // GATHER: one descriptor over all of A; a lane's offset per chunk is its gathered row (beyond every size for rows
    // past the tile's end), the position along k travels in the scalar offset
    uint32_t a_gather[GATHER ? 8 : 1];
    static_assert(!(GATHER && A_KS), "the row gather belongs to the [M][K] form");
    const __amdgpu_buffer_rsrc_t a_all = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.A), 0, static_cast<int>(static_cast<uint32_t>(GATHER ? p.a_rows : 0) * static_cast<uint32_t>(p.lda) * 2u), 0x00020000);
    if constexpr (GATHER) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int r = m0 + 32 * c + (tid >> 3);
            a_gather[c] = r < m_end ? static_cast<uint32_t>(p.a_row_index[r]) * static_cast<uint32_t>(p.lda) * 2u + (tid & 7) * 16u : kOutside;
        }
    }
    // NT with a period: where tile ks of the k range starts in B's columns
    const int b_period = B_KC && p.b_k_period ? p.b_k_period : 0x7fffffff;
    int kb_load = 0;              // ... for the tile the next load_one calls fetch (set by the callers)
    // chunk c (0 .. NA-1: M side, NA .. NA+NB-1: N side) of K-tile ks into its staging register
    auto load_one = [&](int ks, auto cc, uint4 (&ra)[NA], uint4 (&rb)[NB]) {
        constexpr int c = decltype(cc)::value;
        const int k0 = k_begin + ks * TK;
        if constexpr (c < NA) {
            if constexpr (A_KS) {
                ra[c] = load_rows(p.A, p.lda, k0 + 8 * c, k_end, m0, a_lane_ks);
            } else if constexpr (GATHER) {
                const uint32_t off = k0 + (tid & 7) * 8 < k_end ? a_gather[c] : kOutside;
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(a_all, static_cast<int>(off), k0 * 2, 0);
                ra[c] = make_uint4(v.x, v.y, v.z, v.w);
            } else {
                const uint32_t off = k0 + (tid & 7) * 8 < k_end ? a_lane_kc : kOutside;
                ra[c] = load_rows(p.A, p.lda, m0 + 32 * c, m_end, k0, off);
            }
        } else if constexpr (B_KC) {
            const uint32_t off = k0 + (tid & 7) * 8 < k_end ? b_lane_kc : kOutside;
            rb[c - NA] = load_rows(B, p.ldb, n0 + 32 * (c - NA), p.N, kb_load, off);
        } else {
            rb[c - NA] = load_rows(B, p.ldb, k0 + 8 * (c - NA), k_end, n0, b_lane);
        }
    };
    // the same chunk from its staging register into LDS stage `stage`
    auto park_one = [&](int stage, auto cc, const uint4 (&ra)[NA], const uint4 (&rb)[NB]) {
        constexpr int c = decltype(cc)::value;
        uint8_t* as = smem + stage * kStage;
        if constexpr (c < NA) {
            if constexpr (A_KS) {
                *reinterpret_cast<uint4*>(as + ((tid >> 5) + 8 * c) * kPitchM + (tid & 31) * 16) = ra[c];
            } else {
                const int r = (tid >> 3) + 32 * c;
                *reinterpret_cast<uint4*>(as + r * kPitchKC + (((tid & 7) ^ swz(r)) << 4)) = ra[c];
            }
        } else if constexpr (B_KC) {
            const int r = (tid >> 3) + 32 * (c - NA);
            *reinterpret_cast<uint4*>(as + kATile + r * kPitchKC + (((tid & 7) ^ swz(r)) << 4)) = rb[c - NA];
        } else {
            *reinterpret_cast<uint4*>(as + kATile + ((tid >> 5) + 8 * (c - NA)) * kPitchN + (tid & 31) * 16) = rb[c - NA];
        }
    };

    // ---- LDS -> MFMA ----
    v16f acc[4][4];      // [n tile][m tile]
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][i][r] = 0.0f;

    const int frow = lane & 31, khalf = lane >> 5;
    const int ks_n = ks_lane_offset(kPitchN, lane) + wn * 128 * 2, ks_m = ks_lane_offset(kPitchM, lane) + wm * 128 * 2;
    // operand fragments, two sets: k-step s of any K-tile lives in set s % 2
    v8bf nop[2][4], mop[2][4];
    // fragment u (0..3: N side, 4..7: M side) of k-step s of the K-tile in LDS stage `stage`
    auto read_unit = [&](int stage, auto sc, auto uc) {
        constexpr int ks16 = decltype(sc)::value, u = decltype(uc)::value;
        const uint8_t* as = smem + stage * kStage;
        if constexpr (u < 4 && B_KC) {
            const int row = wn * 128 + 32 * u + frow;
            nop[ks16 & 1][u] = *reinterpret_cast<const v8bf*>(as + kATile + row * kPitchKC + (((2 * ks16 + khalf) ^ swz(row)) << 4));
        } else if constexpr (u < 4) {
            nop[ks16 & 1][u] = read_ks<kPitchN>(as + kATile + ks_n, 16 * ks16, 32 * u);
        } else if constexpr (A_KS) {
            mop[ks16 & 1][u - 4] = read_ks<kPitchM>(as + ks_m, 16 * ks16, 32 * (u - 4));
        } else {
            const int row = wm * 128 + 32 * (u - 4) + frow;
            mop[ks16 & 1][u - 4] = *reinterpret_cast<const v8bf*>(as + row * kPitchKC + (((2 * ks16 + khalf) ^ swz(row)) << 4));
        }
    };

    // One K-tile (64 MFMAs per wavefront) with everything else woven between them, one item per MFMA at most (one
    // wavefront per SIMD: whatever waits, the matrix cores wait with it).  While tile ks is multiplied from `stage`:
    //   - the fragments of k-step s + 1 are read during k-step s;
    //   - the 16 loads of tile ks + 2 go out one every fourth MFMA, into the register set tile ks just left;
    //   - tile ks + 1 (requested one tile ago) is parked in the other stage one chunk every third MFMA, done by MFMA 47;
    //   - the barrier follows, and the first fragments of tile ks + 1 are read under the last 16 MFMAs.
    // A tile past the end of the k range is fetched as zeros (it lies beyond the descriptors) and adds nothing, so the
    // loop needs no tail.
    auto ktile = [&](auto stage_c, int ks, uint4 (&ra_new)[NA], uint4 (&rb_new)[NB], const uint4 (&ra_next)[NA], const uint4 (&rb_next)[NB]) {
        constexpr int stage = decltype(stage_c)::value;
        static_for<0, 64>([&](auto mc) {
            constexpr int m = decltype(mc)::value, ks16 = m / 16, q = m % 16;
            acc[q >> 2][q & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nop[ks16 & 1][q >> 2], mop[ks16 & 1][q & 3], acc[q >> 2][q & 3], 0, 0, 0);
            if constexpr (q < 8) {
                if constexpr (ks16 < 3) read_unit(stage, std::integral_constant<int, (ks16 + 1) % 4>{}, std::integral_constant<int, q % 8>{});
                else                    read_unit(stage ^ 1, std::integral_constant<int, 0>{}, std::integral_constant<int, q % 8>{});
            }
            if constexpr (m % 4 == 1) load_one(ks + 2, std::integral_constant<int, m / 4>{}, ra_new, rb_new);
            if constexpr (m < 48 && m % 3 == 2) park_one(stage ^ 1, std::integral_constant<int, (m / 3) % 16>{}, ra_next, rb_next);
            if constexpr (m == 47) __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (B_KC) {          // the next K-tile's loads are one tile further
            kb_load += TK;
            if (kb_load >= b_period) kb_load -= b_period;
        }
    };

    static_assert(NA + NB == 16, "the weave above places 16 loads and 16 LDS stores per K-tile");
    uint4 ra0[NA], rb0[NB], ra1[NA], rb1[NB];
    static_for<0, 16>([&](auto c) { load_one(0, c, ra0, rb0); });
    if constexpr (B_KC) kb_load = TK % b_period;
    static_for<0, 16>([&](auto c) { load_one(1, c, ra1, rb1); });
    if constexpr (B_KC) kb_load = (2 * TK) % b_period;
    static_for<0, 16>([&](auto c) { park_one(0, c, ra0, rb0); });
    __syncthreads();
    static_for<0, 8>([&](auto u) { read_unit(0, std::integral_constant<int, 0>{}, u); });
    for (int ks = 0; ks < nk; ks += 2) {
        ktile(std::integral_constant<int, 0>{}, ks, ra0, rb0, ra1, rb1);
        ktile(std::integral_constant<int, 1>{}, ks + 1, ra1, rb1, ra0, rb0);
    }

    // ---- epilogue: accumulator register r of tile (j, i) is output row m0 + wm*128 + 32 i + lane % 32,
    //      column n0 + wn*128 + 32 j + 8 (r / 4) + 4 (lane / 32) + r % 4 ----
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 128 + 32 * i + frow;
        if (m >= m_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * 128 + 32 * j + 8 * q + 4 * khalf;
                if (n >= p.N) continue;                      // N % 8 == 0: a quad is inside or outside as a whole
                const size_t at = c_base + static_cast<size_t>(m) * p.ldc + n;
                float v[4] = {acc_read(acc[j][i][4 * q]), acc_read(acc[j][i][4 * q + 1]), acc_read(acc[j][i][4 * q + 2]),
                              acc_read(acc[j][i][4 * q + 3])};
                if constexpr (OUT == OUT_STORE_F32) {
                    *reinterpret_cast<float4*>(static_cast<float*>(p.C) + at) = make_float4(v[0], v[1], v[2], v[3]);
                } else if constexpr (OUT == OUT_ACCUM_F32) {
                    float4* dst = reinterpret_cast<float4*>(static_cast<float*>(p.C) + at);
                    float4 c = *dst;
                    c.x += v[0]; c.y += v[1]; c.z += v[2]; c.w += v[3];
                    *dst = c;
                } else {
                    uint2* dst = reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.C) + at);
                    if constexpr (OUT == OUT_ACCUM_BF16) {
                        // fp32 sum of the old value and the product, one rounding (cublasGemmEx with a bf16 C, beta = 1)
                        const uint2 c = *dst;
                        v[0] += bf16_lo(c.x); v[1] += bf16_hi(c.x); v[2] += bf16_lo(c.y); v[3] += bf16_hi(c.y);
                    }
                    *dst = make_uint2(pack_bf16x2_hw(v[0], v[1]), pack_bf16x2_hw(v[2], v[3]));
                }
                // one quad's loads and stores at a time: pulling the whole tile's reads of C to the front would need
                // more registers than the main loop leaves
                if constexpr (OUT == OUT_ACCUM_BF16 || OUT == OUT_ACCUM_F32) __builtin_amdgcn_sched_barrier(0);
            }
    }
}

template <bool A_KS, int OUT, bool GROUPED, bool B_KC = false, bool GATHER = false>
int launch(const BfArgs& p, dim3 grid, hipStream_t st) {
    static std::once_flag once;
    static hipError_t attr = hipSuccess;      // kept: a failed set-up is reported by every call, not only the first
    auto kern = k_gemm_bf16<A_KS, OUT, GROUPED, B_KC, GATHER>;
    std::call_once(once, [&] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    });
    if (attr != hipSuccess) return static_cast<int>(attr);
    kern<<<grid, kThr, kLds, st>>>(p);
    return launch_status();
}

bool operands_ok(const void* A, int lda, const void* B, int ldb, const void* C, int ldc, int c_elem_bytes) {
    return aligned16(A) && aligned16(B) && lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 &&
           (reinterpret_cast<uintptr_t>(C) & (4u * c_elem_bytes - 1u)) == 0;
}

// C[M,N] = A[M,K] . B[K,N]; grouped: per expert over its rows of the compact buffers
int gemm_nn(int M, int N, int K, int E, const int* counts, const int* offsets, const uint16_t* A, int lda, const uint16_t* B,
            int ldb, uint16_t* C, int ldc, void* ws, size_t ws_bytes, bool grouped, cf_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || E < 0) return CF_ERR_INVALID_ARG;
    if (M == 0 || N == 0 || (grouped && E == 0)) return CF_OK;
    if (!A || !B || !C || (grouped && (!counts || !offsets || !ws))) return CF_ERR_INVALID_ARG;
    if (lda < K || ldb < N || ldc < N) return CF_ERR_INVALID_ARG;
    if (N % 8 != 0 || K % 8 != 0 || !operands_ok(A, lda, B, ldb, C, ldc, 2)) return CF_ERR_UNSUPPORTED;
    if (static_cast<size_t>(M) * lda >= (1ull << 30) || static_cast<size_t>(K) * ldb >= (1ull << 30)) return CF_ERR_UNSUPPORTED;
    hipStream_t st = as_stream(stream);
    BfArgs p{};
    p.A = A; p.lda = lda; p.B = B; p.ldb = ldb; p.C = C; p.ldc = ldc;
    p.M = M; p.N = N; p.K = K;
    p.tiles_n = (N + TN - 1) / TN;
    int tiles_m = (M + TM - 1) / TM;
    auto grid_for = [&](int row_tiles) {      // 8 XCDs x the per-XCD share of the tiles, rounded up
        const long long total = static_cast<long long>(row_tiles) * p.tiles_n;
        return dim3(static_cast<unsigned>(8 * ((total + 7) / 8)));
    };
    if (grouped) {
        size_t need = 0;
        cf_fp8_grouped_gemm_workspace_bytes(M, E, &need);
        if (ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 3u)) return CF_ERR_INVALID_ARG;
        tiles_m = M / TM + E;
        build_tile_map(counts, offsets, E, tiles_m, M, static_cast<int*>(ws), st);
        p.counts = counts; p.offsets = offsets;
        p.tile_map = static_cast<const int*>(ws);
        p.b_expert_stride = static_cast<long long>(K) * ldb;
        p.tiles_m = tiles_m;
        return launch<false, OUT_STORE_BF16, true>(p, grid_for(tiles_m), st);
    }
    p.tiles_m = tiles_m;
    return launch<false, OUT_STORE_BF16, false>(p, grid_for(tiles_m), st);
}

// C[M,N] += A[K,M]^T . B[K,N]; grouped: per expert, K running over its rows of the compact buffers, C[E,M,N]
template <int OUT>
int gemm_tn(int M, int N, int K, int E, const int* counts, const int* offsets, const uint16_t* A, int lda, const uint16_t* B,
            int ldb, void* C, int ldc, bool grouped, cf_stream_t stream) {
    if (M < 0 || N < 0 || K < 0 || E < 0) return CF_ERR_INVALID_ARG;
    if (M == 0 || N == 0 || K == 0 || (grouped && E == 0)) return CF_OK;
    if (!A || !B || !C || (grouped && (!counts || !offsets))) return CF_ERR_INVALID_ARG;
    if (lda < M || ldb < N || ldc < N) return CF_ERR_INVALID_ARG;
    if (N % 8 != 0 || M % 8 != 0 || !operands_ok(A, lda, B, ldb, C, ldc, OUT == OUT_ACCUM_F32 ? 4 : 2)) return CF_ERR_UNSUPPORTED;
    if (static_cast<size_t>(K) * lda >= (1ull << 30) || static_cast<size_t>(K) * ldb >= (1ull << 30)) return CF_ERR_UNSUPPORTED;
    hipStream_t st = as_stream(stream);
    BfArgs p{};
    p.A = A; p.lda = lda; p.B = B; p.ldb = ldb; p.C = C; p.ldc = ldc;
    p.M = M; p.N = N; p.K = K;
    p.tiles_n = (N + TN - 1) / TN;
    p.tiles_m = (M + TM - 1) / TM;
    const long long tiles = static_cast<long long>(p.tiles_m) * p.tiles_n;
    if (grouped) {
        p.counts = counts; p.offsets = offsets;
        p.num_experts = E;
        p.c_expert_stride = static_cast<long long>(M) * ldc;
        const long long blocks = 8LL * ((E + 7) / 8) * tiles;
        if (blocks >= (1LL << 31)) return CF_ERR_UNSUPPORTED;
        return launch<true, OUT, true>(p, dim3(static_cast<unsigned>(blocks)), st);
    }
    return launch<true, OUT, false>(p, dim3(static_cast<unsigned>(8 * ((tiles + 7) / 8))), st);
}

}  // namespace

// C[r, :] = sum over terms t of A[r, t*Kb : (t+1)*Kb] . B[expert(r)]^T: the forward-pass form, A [total_rows, terms*Kb]
// with its rows grouped by expert (or, with d_a_row_index, gathered from the a_rows rows of A: compact row r is row
// d_a_row_index[r]), B [num_experts, N, Kb] as a weight matrix lies in memory, C bf16 or fp32 [total, N];
// d_tile_map is the table build_tile_map made for these counts.  Kb % 8 == 0 (% 64 with several terms), N % 8 == 0.
int grouped_gemm_bf16_nt(int total_rows, int N, int Kb, int terms, int num_experts, const uint16_t* A, int a_rows, int lda,
                         const int* d_a_row_index, const uint16_t* B, void* C, int ldc, bool c_is_f32, const int* d_tile_map,
                         cf_stream_t stream) {
    if (total_rows <= 0 || N <= 0 || num_experts <= 0) return CF_OK;
    if (!A || !B || !C || !d_tile_map || terms < 1 || a_rows < 0) return CF_ERR_INVALID_ARG;
    const long long K = static_cast<long long>(terms) * Kb;
    if ((terms > 1 ? Kb % kMaxTK : Kb % 8) != 0 || Kb <= 0 || lda < K || ldc < N || N % 8 != 0 || !operands_ok(A, lda, B, Kb, C, ldc, c_is_f32 ? 4 : 2) ||
        static_cast<size_t>(d_a_row_index ? a_rows : total_rows) * lda >= (1ull << 30) || static_cast<size_t>(N) * Kb >= (1ull << 30))
        return CF_ERR_UNSUPPORTED;
    BfArgs p{};
    p.A = A; p.lda = lda; p.B = B; p.ldb = Kb; p.C = C; p.ldc = ldc;
    p.M = total_rows; p.N = N; p.K = static_cast<int>(K);
    p.tiles_n = (N + TN - 1) / TN;
    p.tiles_m = total_rows / TM + num_experts;
    p.tile_map = d_tile_map;
    p.b_expert_stride = static_cast<long long>(N) * Kb;
    p.b_k_period = terms > 1 ? Kb : 0;
    p.a_row_index = d_a_row_index;
    p.a_rows = a_rows;
    const long long total = static_cast<long long>(p.tiles_m) * p.tiles_n;
    const dim3 grid(static_cast<unsigned>(8 * ((total + 7) / 8)));
    hipStream_t st = as_stream(stream);
    if (d_a_row_index) {
        if (!c_is_f32) return CF_ERR_UNSUPPORTED;      // the one caller stores fp32
        return launch<false, OUT_STORE_F32, true, true, true>(p, grid, st);
    }
    return c_is_f32 ? launch<false, OUT_STORE_F32, true, true>(p, grid, st) : launch<false, OUT_STORE_BF16, true, true>(p, grid, st);
}
}  // namespace cf

using namespace cf;

extern "C" {

int cf_gemm_bf16_nn(int M, int N, int K, const uint16_t* A, int lda, const uint16_t* B, int ldb, uint16_t* C, int ldc,
                    cf_stream_t stream) {
    return gemm_nn(M, N, K, 0, nullptr, nullptr, A, lda, B, ldb, C, ldc, nullptr, 0, false, stream);
}
int cf_gemm_bf16_tn_accum_f32(int M, int N, int K, const uint16_t* A, int lda, const uint16_t* B, int ldb, float* C, int ldc,
                              cf_stream_t stream) {
    return gemm_tn<OUT_ACCUM_F32>(M, N, K, 0, nullptr, nullptr, A, lda, B, ldb, C, ldc, false, stream);
}
int cf_gemm_bf16_tn_accum_bf16(int M, int N, int K, const uint16_t* A, int lda, const uint16_t* B, int ldb, uint16_t* C,
                               int ldc, cf_stream_t stream) {
    return gemm_tn<OUT_ACCUM_BF16>(M, N, K, 0, nullptr, nullptr, A, lda, B, ldb, C, ldc, false, stream);
}
int cf_moe_grouped_gemm_bf16_nn(int total_rows, int N, int K, int num_experts, const int* d_counts, const int* d_offsets,
                                const uint16_t* A, int lda, const uint16_t* B, uint16_t* C, int ldc, void* d_workspace,
                                size_t workspace_bytes, cf_stream_t stream) {
    return gemm_nn(total_rows, N, K, num_experts, d_counts, d_offsets, A, lda, B, N, C, ldc, d_workspace, workspace_bytes, true,
                   stream);
}
int cf_moe_grouped_gemm_bf16_tn_accum_f32(int M, int N, int total_rows, int num_experts, const int* d_counts,
                                          const int* d_offsets, const uint16_t* A, int lda, const uint16_t* B, int ldb,
                                          float* C, cf_stream_t stream) {
    return gemm_tn<OUT_ACCUM_F32>(M, N, total_rows, num_experts, d_counts, d_offsets, A, lda, B, ldb, C, N, true, stream);
}
int cf_moe_grouped_gemm_bf16_tn_accum_bf16(int M, int N, int total_rows, int num_experts, const int* d_counts,
                                           const int* d_offsets, const uint16_t* A, int lda, const uint16_t* B, int ldb,
                                           uint16_t* C, cf_stream_t stream) {
    return gemm_tn<OUT_ACCUM_BF16>(M, N, total_rows, num_experts, d_counts, d_offsets, A, lda, B, ldb, C, N, true, stream);
}

}  // extern "C"
