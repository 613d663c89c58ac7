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
// column i.  Two such reads give a lane its eight k of a 16x16x32 MFMA operand (lanes 16 g .. 16 g + 15 hold k rows
// 8 g .. 8 g + 7 of a 32-deep k-step).  An operand that is K-contiguous in memory takes the usual path (128-byte LDS
// rows, 16-byte chunks xor-swizzled, ds_read_b128).
//
// Workgroup tile 256 (M) x 256 (N) x 64 (K), four wavefronts 2 x 2, each 128 x 128 = 8 x 8 blocks of
// v_mfma_f32_16x16x32_bf16 with fp32 accumulators (four registers per block).  Both bf16 MFMA shapes do 1024 FLOP per
// cycle and SIMD; at the socket power limit, where these GEMMs run, the 16 x 16 x 32 shape delivers 14 % more (MFMAs
// alone on random operands, probes/mfma_shape_power_bf16.hip).  The N-side operand goes to the MFMA "A" side, so a lane
// ends up with four consecutive output columns of one output row per block.  Global loads are register staged two
// K-tiles ahead (16 bytes per lane), LDS is double buffered, one barrier per K-tile.
// Operand registers: four sets of four blocks (N halves N0, N1; M halves M0, M1; 16 registers each).  A 32-deep k-step
// is four phases of sixteen MFMAs, (N0, M[p]) -> (N0, M[1-p]) -> (N1, M[1-p]) -> (N1, M[p]) with p the k-step's parity,
// and the set a phase leaves behind is refilled two phases before it is needed again: M[1-p] and N1 of this k-step
// under phases 0 and 1, N0 and M[1-p] of the next k-step under phases 2 and 3.  A K-tile is two k-steps.
// Rows, columns and k beyond the operands' bounds are read as zeros (buffer loads with the operand's size in their
// descriptor), so any n_e works.
// The kernel is persistent: one workgroup per CU walks a sequence of output tiles with the operand fetch running on
// across the tile boundaries, and writes a finished tile through LDS in whole 256-byte (bf16) or 512-byte (fp32) row
// pieces.  Per output tile that leaves about 14 thousand cycles beside the K-tiles (11 of them the stores' way to memory)
// where one workgroup per tile with stores straight from the accumulator layout took 27 thousand.
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
typedef float v4f __attribute__((ext_vector_type(4)));
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

// 16-byte chunk swizzle of a K-contiguous tile: a ds_read_b128 of a 16 x 16 x 32 operand has rows 0-7 of k-group g go
// with rows 8-15 of k-group g ^ 1 (chunks g and g ^ 1 of the k-step), and the 16 lanes must hit 16 different 16-byte
// slots of a 256-byte line
__device__ __forceinline__ int swz(int row) { return (row ^ (((row >> 3) & 1) << 1)) & 7; }

// Eight k of one column for every lane: two transposing reads of a [k][columns] tile.  `lane_ptr` is the tile's base
// plus this lane's share of the address (ks_lane_offset); the k-step and the column block are compile-time
// constants, so they end up in the instructions' immediate offsets and no address register is spent on them.
// k rows 8 .. 15 (mod 16) of a [k][columns] tile are parked 32 bytes to the right (into the row's pad), so that the
// k-groups that one instruction serves together do not meet on the same banks.
__device__ __forceinline__ int ks_lane_offset(int pitch, int lane) {
    const int g = lane >> 4, r = lane & 15;
    return (8 * g + (r >> 2)) * pitch + (g & 1) * 32 + 4 * (r & 3) * 2;
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

    // ---- which tiles ----
    // Persistent: one workgroup per CU walks a sequence of output tiles, and the operand fetch runs on across the tile
    // boundaries (the last two K-tiles of a tile already request the first two of the next), so only the first tile of a
    // workgroup waits for memory with idle matrix cores.
    // Workgroups go to the 8 XCDs round-robin (launch position % 8), each XCD with its own 4 MiB L2.  Position b is
    // therefore read as (XCD x = b % 8, that XCD's i-th workgroup), and what an XCD runs at one time is made to share
    // operands: in the row-major forms XCD x walks the contiguous range [x * per, (x + 1) * per) of the tile order in
    // patches of 8 row tiles x 4 column tiles, its workgroups taking every (grid / 8)-th tile of it; in the grouped
    // weight-gradient form XCD x owns experts x, x + 8, ... whole, so that all tiles of an expert stream the same rows
    // through one L2.
    const int x = blockIdx.x % 8, xi_step = gridDim.x / 8;
    constexpr int TK = 64;
    constexpr int NA = A_KS ? TK / 8 : 8, NB = TK / 8;       // 16-byte chunks per lane and K-tile
    constexpr uint32_t kOutside = 0x80000000u;
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    int row_tiles = p.tiles_m;
    if constexpr (GROUPED && !A_KS) row_tiles = __builtin_amdgcn_readfirstlane(p.tile_map[0]);
    const int total = row_tiles * p.tiles_n, per = (total + 7) / 8;     // the row-major forms
    const int tiles_mn = p.tiles_m * p.tiles_n;                          // the grouped weight-gradient form: per expert

    struct Tile {
        int m0, n0, m_end, k_begin, k_end;
        int nk2;                // K-tiles, rounded up to an even number (at least two): the pad tile lies beyond the k range
        long long b_off;        // elements from p.B to the expert's matrix
        size_t c_base;
        bool valid;
    };
    // The grouped forms read what they need of a tile from memory (its row of the tile table, or the expert's offset
    // and count).  That read is issued one tile before its values are used, through buffer loads whose offsets lie
    // beyond the descriptor for positions past the end of the sequence: no branch, no wait.
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t rs_map = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int*>(GROUPED && !A_KS ? p.tile_map : nullptr), 0, GROUPED && !A_KS ? (1 + 5 * p.tiles_m) * 4 : 0, 0x00020000);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t rs_offsets = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int*>(GROUPED && A_KS ? p.offsets : nullptr), 0, GROUPED && A_KS ? p.num_experts * 4 : 0, 0x00020000);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t rs_counts = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int*>(GROUPED && A_KS ? p.counts : nullptr), 0, GROUPED && A_KS ? p.num_experts * 4 : 0, 0x00020000);
    // position xi of this XCD's sequence -> (valid, row tile, first column) for the row-major forms
    auto place = [&](int xi, int& tmi, int& n0) {
        const int t = x * per + xi;
        const bool valid = xi < per && t < total;
        constexpr int GM = 8;
        const int tt = valid ? t : 0;
        const int group = tt / (GM * p.tiles_n), first = group * GM;
        const int gm = max(min(GM, row_tiles - first), 1), in_group = tt - group * GM * p.tiles_n;
        tmi = first + in_group % gm;
        n0 = (in_group / gm) * TN;
        return valid;
    };
    auto fetch = [&](int xi) {
        int2 rec = make_int2(0, 0);
        if constexpr (GROUPED && A_KS) {
            const int e = x + 8 * (xi / tiles_mn);
            const uint32_t off = e < p.num_experts ? static_cast<uint32_t>(e) * 4u : kOutside;
            rec.x = __builtin_amdgcn_raw_buffer_load_b32(rs_offsets, static_cast<int>(off), 0, 0);
            rec.y = __builtin_amdgcn_raw_buffer_load_b32(rs_counts, static_cast<int>(off), 0, 0);
        } else if constexpr (GROUPED) {
            int tmi, n0;
            const bool valid = place(xi, tmi, n0);
            const uint32_t off = valid && lane < 5 ? static_cast<uint32_t>(1 + 5 * tmi + lane) * 4u : kOutside;
            rec.x = __builtin_amdgcn_raw_buffer_load_b32(rs_map, static_cast<int>(off), 0, 0);     // lane l: word l of the row
        }
        return rec;
    };
    auto decode = [&](int xi, int2 rec) {
        Tile t{};
        if constexpr (GROUPED && A_KS) {
            const int e = x + 8 * (xi / tiles_mn), ti = xi % tiles_mn;
            t.valid = e < p.num_experts;
            t.m0 = (ti % p.tiles_m) * TM;
            t.n0 = (ti / p.tiles_m) * TN;
            t.m_end = p.M;
            // an expert's row range is cut at the rows the compact buffers hold (p.K), as the tile table cuts it
            t.k_begin = min(max(__builtin_amdgcn_readfirstlane(rec.x), 0), p.K);
            t.k_end = min(t.k_begin + max(__builtin_amdgcn_readfirstlane(rec.y), 0), p.K);
            t.c_base = static_cast<size_t>(t.valid ? e : 0) * p.c_expert_stride;
        } else {
            int tmi;
            t.valid = place(xi, tmi, t.n0);
            t.m0 = tmi * TM;
            t.m_end = p.M;
            t.k_end = p.K;
            if constexpr (GROUPED) {
                const int expert = __builtin_amdgcn_readlane(rec.x, 0), first_row = __builtin_amdgcn_readlane(rec.x, 1);
                const int end_row = __builtin_amdgcn_readlane(rec.x, 2), first_tile = __builtin_amdgcn_readlane(rec.x, 3);
                t.m0 = first_row + (tmi - first_tile) * TM;
                t.m_end = min(t.m0 + TM, end_row);
                t.b_off = static_cast<long long>(expert) * p.b_expert_stride;
            }
        }
        if (!t.valid) {         // a position past the end: every load of it lies beyond its descriptor
            t.m0 = t.n0 = t.m_end = t.k_begin = t.k_end = 0;
            t.b_off = 0;
            t.c_base = 0;
        }
        const int nk = (max(t.k_end - t.k_begin, 0) + TK - 1) / TK;
        t.nk2 = max((nk + 1) & ~1, 2);
        return t;
    };

    // ---- global -> registers -> LDS: 16-byte chunks through buffer loads ----
    // A buffer load takes a descriptor with a base and a size in bytes and returns zeros for a lane whose offset lies
    // beyond the size, so every load is issued unconditionally (loads under branches would keep the compiler from
    // counting the loads in flight: it would wait for all of them, the prefetch included, before the first LDS store)
    // and the zero fill of the ragged ends costs nothing.  Each operand gets one descriptor per K-tile, built with scalar
    // instructions: the base is the tile's first row (and first k), the size what is left of the operand from there
    // (nothing, past the end of the k range).  A lane's offset is its row within the first eight-row (32-row) group and
    // its 16-byte column, plus the group's distance from the tile's first row; a lane whose columns lie outside the
    // operand (or, for the K-contiguous form, whose k chunk lies beyond K) starts from an offset beyond every size.
    // The launcher keeps operands below 2 GiB, so the sum does not wrap.  (A descriptor per load costs about ten
    // scalar instructions in front of one MFMA in every eight, more than the MFMA's 16 cycles cover.)
    // rows [row0, row_end) of a row-major operand with `ld` elements per row, seen from element `col0` of row row0
    auto rows_rsrc = [](const uint16_t* base, int ld, int row0, int row_end, int col0) {
        const int rows_left = max(row_end - row0, 0);
        return __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(base + static_cast<size_t>(row0) * ld + col0), 0,
            static_cast<int>(static_cast<uint32_t>(rows_left) * static_cast<uint32_t>(ld) * 2u), 0x00020000);
    };
    auto load_at = [](__amdgpu_buffer_rsrc_t rs, uint32_t off) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<int>(off), 0, 0);
        return make_uint4(v.x, v.y, v.z, v.w);
    };
    // [k][columns] operands: this lane's row within a group of eight k rows and its 16-byte column
    const uint32_t b_lane_ks = (tid >> 5) * static_cast<uint32_t>(p.ldb) * 2u + (tid & 31) * 16u;
    const uint32_t a_lane_ks = (tid >> 5) * static_cast<uint32_t>(p.lda) * 2u + (tid & 31) * 16u;
    // [m][k] operand: this lane's row within a group of 32 rows and its 16-byte k chunk
    const uint32_t a_lane_kc = (tid >> 3) * static_cast<uint32_t>(p.lda) * 2u + (tid & 7) * 16u;
    const uint32_t b_lane_kc = (tid >> 3) * static_cast<uint32_t>(p.ldb) * 2u + (tid & 7) * 16u;
    // GATHER: one descriptor over all of A; a lane's offset per chunk is its gathered row (beyond every size for rows
    // past the tile's end), the position along k travels in the scalar offset.  The row index is itself read through
    // a descriptor, one tile before the rows are.
    static_assert(!(GATHER && A_KS), "the row gather belongs to the [M][K] form");
    const __amdgpu_buffer_rsrc_t a_all = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.A), 0, static_cast<int>(static_cast<uint32_t>(GATHER ? p.a_rows : 0) * static_cast<uint32_t>(p.lda) * 2u), 0x00020000);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t rs_index = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int*>(GATHER ? p.a_row_index : nullptr), 0, GATHER ? p.M * 4 : 0, 0x00020000);
    constexpr int NG = GATHER ? 8 : 1;
    auto gather_rows = [&](const Tile& t, int (&rows)[NG]) {       // the index values, as loaded
        if constexpr (GATHER) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int r = t.m0 + 32 * c + (tid >> 3);
                rows[c] = __builtin_amdgcn_raw_buffer_load_b32(rs_index, static_cast<int>(r < t.m_end ? static_cast<uint32_t>(r) * 4u : kOutside), 0, 0);
            }
        }
    };
    auto gather_offsets = [&](const Tile& t, const int (&rows)[NG], uint32_t (&offs)[NG]) {
        if constexpr (GATHER) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int r = t.m0 + 32 * c + (tid >> 3);
                offs[c] = r < t.m_end ? static_cast<uint32_t>(rows[c]) * static_cast<uint32_t>(p.lda) * 2u + (tid & 7) * 16u : kOutside;
            }
        }
    };

    // ---- the fetch cursor: K-tile lks of tile L, two K-tiles ahead of the MFMAs ----
    // L_after is the tile after L (decoded a tile ahead, so that its gathered row numbers can be on their way), rec_next
    // the record of the tile after that; L_before is the tile L came from: when the MFMAs finish a tile, the fetch is in
    // the next one or, if that has two K-tiles only, already in the one after it (tiles_ahead says which).
    const int b_period = B_KC && p.b_k_period ? p.b_k_period : 0x7fffffff;
    int xi_next = blockIdx.x / 8;
    Tile L = decode(xi_next, fetch(xi_next));
    if (!L.valid) return;
    xi_next += xi_step;
    Tile L_after = decode(xi_next, fetch(xi_next));
    xi_next += xi_step;
    int2 rec_next = fetch(xi_next);
    Tile L_before = L;
    int tiles_ahead = 0;
    int lks = 0;
    int kb_load = 0;              // NT with a period: where K-tile lks starts in B's columns
    uint32_t a_gather[NG];
    int rows_after[NG];
    {
        int rows_now[NG];
        gather_rows(L, rows_now);
        gather_offsets(L, rows_now, a_gather);
        gather_rows(L_after, rows_after);
    }
    // to the next K-tile, after the 16 loads of one.  Tiles have an even number of K-tiles and the cursor starts on an
    // even one, so only the step off an odd K-tile (END_OF_PAIR) can leave the tile: the other needs no branch.
    auto advance = [&](auto end_of_pair) {
        ++lks;
        if constexpr (B_KC) {
            kb_load += TK;
            if (kb_load >= b_period) kb_load -= b_period;
        }
        if constexpr (!decltype(end_of_pair)::value) return;
        if (lks == L.nk2) {
            L_before = L;
            L = L_after;
            gather_offsets(L, rows_after, a_gather);
            L_after = decode(xi_next, rec_next);
            xi_next += xi_step;
            rec_next = fetch(xi_next);
            gather_rows(L_after, rows_after);
            ++tiles_ahead;
            lks = 0;
            kb_load = 0;
        }
    };
    // One descriptor per operand and K-tile, built by the tile's first load of that operand; the chunks of the tile
    // differ in the lane offset only (one vector add each).
    __amdgpu_buffer_rsrc_t rs_a = a_all, rs_b = a_all;
    uint32_t off_a = kOutside, off_b = kOutside;
    const uint32_t a_step = (A_KS ? 8u : 32u) * static_cast<uint32_t>(p.lda) * 2u;
    const uint32_t b_step = (B_KC ? 32u : 8u) * static_cast<uint32_t>(p.ldb) * 2u;
    // chunk c (0 .. NA-1: M side, NA .. NA+NB-1: N side) of the cursor's K-tile into its staging register
    auto load_one = [&](auto cc, uint4 (&ra)[NA], uint4 (&rb)[NB]) {
        constexpr int c = decltype(cc)::value;
        const int k0 = L.k_begin + lks * TK;
        if constexpr (c == 0 && !GATHER) {
            if constexpr (A_KS) {
                rs_a = rows_rsrc(p.A, p.lda, k0, L.k_end, L.m0);
                off_a = L.m0 + (tid & 31) * 8 < p.M ? a_lane_ks : kOutside;
            } else {
                rs_a = rows_rsrc(p.A, p.lda, L.m0, L.m_end, k0);
                off_a = k0 + (tid & 7) * 8 < L.k_end ? a_lane_kc : kOutside;
            }
        }
        if constexpr (c == NA) {
            const uint16_t* B = p.B + L.b_off;
            if constexpr (B_KC) {
                rs_b = rows_rsrc(B, p.ldb, L.n0, p.N, kb_load);
                off_b = k0 + (tid & 7) * 8 < L.k_end ? b_lane_kc : kOutside;
            } else {
                rs_b = rows_rsrc(B, p.ldb, k0, L.k_end, L.n0);
                off_b = L.n0 + (tid & 31) * 8 < p.N ? b_lane_ks : kOutside;
            }
        }
        if constexpr (c < NA) {
            if constexpr (GATHER) {
                const uint32_t off = k0 + (tid & 7) * 8 < L.k_end ? a_gather[c] : kOutside;
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(a_all, static_cast<int>(off), k0 * 2, 0);
                ra[c] = make_uint4(v.x, v.y, v.z, v.w);
            } else {
                ra[c] = load_at(rs_a, off_a + c * a_step);
            }
        } else {
            rb[c - NA] = load_at(rs_b, off_b + (c - NA) * b_step);
        }
    };
    // the same chunk from its staging register into LDS stage `stage`
    auto park_one = [&](int stage, auto cc, const uint4 (&ra)[NA], const uint4 (&rb)[NB]) {
        constexpr int c = decltype(cc)::value;
        uint8_t* as = smem + stage * kStage;
        if constexpr (c < NA) {
            if constexpr (A_KS) {
                *reinterpret_cast<uint4*>(as + ((tid >> 5) + 8 * c) * kPitchM + (c & 1) * 32 + (tid & 31) * 16) = ra[c];
            } else {
                const int r = (tid >> 3) + 32 * c;
                *reinterpret_cast<uint4*>(as + r * kPitchKC + (((tid & 7) ^ swz(r)) << 4)) = ra[c];
            }
        } else if constexpr (B_KC) {
            const int r = (tid >> 3) + 32 * (c - NA);
            *reinterpret_cast<uint4*>(as + kATile + r * kPitchKC + (((tid & 7) ^ swz(r)) << 4)) = rb[c - NA];
        } else {
            *reinterpret_cast<uint4*>(as + kATile + ((tid >> 5) + 8 * (c - NA)) * kPitchN + ((c - NA) & 1) * 32 + (tid & 31) * 16) = rb[c - NA];
        }
    };

    // ---- LDS -> MFMA ----
    v4f acc[8][8];      // [n block][m block]
    auto clear_acc = [&] {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[j][i][r] = 0.0f;
    };
    clear_acc();

    const int r16 = lane & 15, kg = lane >> 4;
    const int ks_n = ks_lane_offset(kPitchN, lane) + wn * 128 * 2, ks_m = ks_lane_offset(kPitchM, lane) + wm * 128 * 2;
    // K-contiguous tiles: this lane's row within a block and its chunk for either k-step (the swizzle depends on the
    // row modulo 16 only, so the block is an immediate offset)
    int kc[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) kc[s2] = r16 * kPitchKC + (((4 * s2 + kg) ^ swz(r16)) << 4);
    // operand sets: [half of the wavefront's 128 columns / rows][block]
    v8bf nset[2][4], mset[2][4];
    // block R (0..3) of set SET (0, 1: N halves; 2, 3: M halves) for k-step S of the K-tile in LDS stage `stage`: one
    // ds_read_b128 of a K-contiguous operand, two transposing reads (k rows + 0 .. 3 and + 4 .. 7) of a [k][columns] one
    auto read_set = [&](int stage, auto sc, auto setc, auto rc_) {
        constexpr int S = decltype(sc)::value, SET = decltype(setc)::value, R = decltype(rc_)::value;
        const uint8_t* as = smem + stage * kStage;
        constexpr bool NSIDE = SET < 2;
        constexpr bool KC = NSIDE ? B_KC : !A_KS;
        constexpr int half = SET & 1, blk = half * 4 + R;
        v8bf v;
        if constexpr (KC) {
            const uint8_t* base = as + (NSIDE ? kATile + wn * 128 * kPitchKC : wm * 128 * kPitchKC);
            v = *reinterpret_cast<const v8bf*>(base + blk * 16 * kPitchKC + kc[S]);
        } else {
            constexpr int PITCH = NSIDE ? kPitchN : kPitchM;
            const uint8_t* pl = as + (NSIDE ? kATile + ks_n : ks_m) + 32 * S * PITCH + 16 * blk * 2;
            const v4bf lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4bf_ptr)(pl));
            const v4bf hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4bf_ptr)(pl + 4 * PITCH));
            v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        if constexpr (NSIDE) nset[half][R] = v; else mset[half][R] = v;
    };
    constexpr int RN = 4, RM = 4;       // read_set calls per set

    // The forms that add to C read it in the epilogue, with idle matrix cores: a round trip to HBM per pass.  Under the
    // tile's last pair of K-tiles every 128-byte line of the wavefront's 128 x 128 block of C is therefore touched once
    // (one dword per lane, distinct lines), so that the epilogue's reads find it in the L2 / the memory-side cache.
    // The touches are issued in every pair, from offsets beyond the descriptor in all but the last.
    constexpr bool ACCUM = OUT == OUT_ACCUM_BF16 || OUT == OUT_ACCUM_F32;
    constexpr int CE = OUT == OUT_ACCUM_F32 || OUT == OUT_STORE_F32 ? 4 : 2;        // bytes per element of C
    constexpr int NTOUCH = ACCUM ? 2 * CE : 1;              // 128 rows x CE lines / 64 lanes
    [[maybe_unused]] int touched[NTOUCH] = {};
    [[maybe_unused]] __amdgpu_buffer_rsrc_t rs_c = a_all;
    [[maybe_unused]] bool touch_ok = false;
    [[maybe_unused]] const uint32_t touch_lane = (lane / CE) * static_cast<uint32_t>(p.ldc) * CE + (lane % CE) * 128u;
    [[maybe_unused]] const uint32_t touch_step = (64 / CE) * static_cast<uint32_t>(p.ldc) * CE;
    [[maybe_unused]] auto touch_one = [&](auto tc) {
        constexpr int t = decltype(tc)::value;
        touched[t] = __builtin_amdgcn_raw_buffer_load_b32(rs_c, static_cast<int>(touch_ok ? touch_lane + t * touch_step : kOutside), 0, 0);
    };
    // the wavefront's block of the output tile `t`, rows beyond the tile's end cut off
    [[maybe_unused]] auto c_block_rsrc = [&](const Tile& t) {
        const int row_w = t.m0 + wm * 128;
        const int rows = min(max(t.m_end - row_w, 0), 128);
        return __builtin_amdgcn_make_buffer_rsrc(
            static_cast<uint8_t*>(p.C) + (t.c_base + static_cast<size_t>(row_w) * p.ldc + t.n0 + wn * 128) * CE, 0,
            static_cast<int>(static_cast<uint32_t>(rows) * static_cast<uint32_t>(p.ldc) * CE), 0x00020000);
    };

    // One K-tile: two k-steps of four phases, 128 MFMAs per wavefront, with everything else woven between them (one
    // wavefront per SIMD: whatever waits, the matrix cores wait with it).  While tile ks is multiplied from `stage`:
    //   - a phase refills the set the phase before it left behind (see the top of the file);
    //   - the 16 loads of tile ks + 2 (the fetch cursor's) go out one every eighth MFMA, into the register set tile ks just left;
    //   - tile ks + 1 (requested one tile ago) is parked in the other stage three chunks per phase, done by MFMA 83;
    //   - the barrier follows MFMA 95, and the first sets of tile ks + 1 are read under the last 32 MFMAs.
    // A tile past the end of the k range is fetched as zeros (it lies beyond the descriptors) and adds nothing, so the
    // loop needs no tail; past the last K-tile of an output tile, "tile ks + 1" is the first of the next output tile.
    auto ktile = [&](auto stage_c, uint4 (&ra_new)[NA], uint4 (&rb_new)[NB], const uint4 (&ra_next)[NA], const uint4 (&rb_next)[NB]) {
        constexpr int stage = decltype(stage_c)::value;
        static_for<0, 128>([&](auto mc) {
            constexpr int m = decltype(mc)::value, S = m / 64, ph = (m % 64) / 16, q = m % 16;
            // k-step S has parity S: phases (N0, M[S]), (N0, M[1-S]), (N1, M[1-S]), (N1, M[S])
            constexpr int nh = ph >> 1, mh = (ph == 0 || ph == 3) ? S : 1 - S;
            constexpr int jn = nh * 4 + (q >> 2), im = mh * 4 + (q & 3);
            // issued through inline assembly with the accumulator tied to the destination: left to the compiler, the 64
            // four-register accumulators come out of a K-tile in other registers than they went in and are moved back
            // through the vector ALU at the loop's end (several hundred moves per K-tile pair)
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[jn][im]) : "v"(nset[nh][q >> 2]), "v"(mset[mh][q & 3]));
            // refills: ph 0: M[1-S] of this k-step; ph 1: N1 of this k-step; ph 2: N0 of the next k-step; ph 3: M[1-S] of the next
            if constexpr (ph == 0) {
                if constexpr (q < 2 * RM && q % 2 == 0) read_set(stage, std::integral_constant<int, S>{}, std::integral_constant<int, 2 + (1 - S)>{}, std::integral_constant<int, (q / 2) % RM>{});
            } else if constexpr (ph == 1) {
                if constexpr (q < 2 * RN && q % 2 == 0) read_set(stage, std::integral_constant<int, S>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, (q / 2) % RN>{});
            } else if constexpr (ph == 2) {
                if constexpr (q < 2 * RN && q % 2 == 0) read_set(S == 0 ? stage : stage ^ 1, std::integral_constant<int, 1 - S>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, (q / 2) % RN>{});
            } else {
                if constexpr (q < 2 * RM && q % 2 == 0) read_set(S == 0 ? stage : stage ^ 1, std::integral_constant<int, 1 - S>{}, std::integral_constant<int, 2 + (1 - S)>{}, std::integral_constant<int, (q / 2) % RM>{});
            }
            if constexpr (m % 8 == 7) load_one(std::integral_constant<int, m / 8>{}, ra_new, rb_new);
            if constexpr (ACCUM && stage == 0 && m % 8 == 1 && m / 8 < NTOUCH) touch_one(std::integral_constant<int, m / 8>{});
            // three LDS stores per sixteen MFMAs, after MFMAs that have neither an operand read nor a load behind them
            constexpr int park = 3 * (m / 16) + (q == 3 ? 0 : q == 10 ? 1 : 2);
            if constexpr ((q == 3 || q == 10 || q == 13) && park < 16) park_one(stage ^ 1, std::integral_constant<int, park % 16>{}, ra_next, rb_next);
            if constexpr (m == 95) __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
        });
        advance(std::integral_constant<bool, stage == 1>{});
    };

    static_assert(NA + NB == 16, "the weave above places 16 loads and 16 LDS stores per K-tile");
    uint4 ra0[NA], rb0[NB], ra1[NA], rb1[NB];
    Tile cur = L;
    static_for<0, 16>([&](auto c) { load_one(c, ra0, rb0); });
    advance(std::false_type{});
    static_for<0, 16>([&](auto c) { load_one(c, ra1, rb1); });
    advance(std::true_type{});
    static_for<0, 16>([&](auto c) { park_one(0, c, ra0, rb0); });
    __syncthreads();
    // the first k-step (parity 0) starts with (N0, M0)
    static_for<0, RN>([&](auto r) { read_set(0, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, r); });
    static_for<0, RM>([&](auto r) { read_set(0, std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{}, r); });
    while (true) {
        if constexpr (ACCUM) rs_c = c_block_rsrc(cur);
        for (int ks = 0; ks < cur.nk2; ks += 2) {
            if constexpr (ACCUM) touch_ok = ks + 2 >= cur.nk2 && cur.n0 + wn * 128 + (lane % CE) * (128 / CE) < p.N;
            ktile(std::integral_constant<int, 0>{}, ra0, rb0, ra1, rb1);
            ktile(std::integral_constant<int, 1>{}, ra1, rb1, ra0, rb0);
        }
        // the MFMAs above are opaque to the compiler's hazard handling: leave the wait states between the last of them
        // and the first read of an accumulator explicitly
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
        // ---- epilogue: accumulator register q of block (j, i) is output row m0 + wm*128 + 16 i + lane % 16,
        //      column n0 + wn*128 + 16 j + 4 (lane / 16) + q.  Written from there a store instruction would cover sixteen
        //      rows with 32 bytes each; instead the wavefront turns its 128 x 128 outputs round in LDS, 64 rows (bf16) or
        //      32 rows (fp32) at a time, and stores (or adds to) whole 256-byte / 512-byte row pieces.  The staging area
        //      is the wavefront's quarter of LDS stage 1: every output tile ends on that stage, nobody reads it after
        //      the last K-tile's barrier, and nobody parks into it before the barrier below.
        //      An empty k range adds nothing (and must not turn a -0 of C into +0). ----
        const bool nothing_to_add = (OUT == OUT_ACCUM_BF16 || OUT == OUT_ACCUM_F32) && cur.k_end <= cur.k_begin;
        if constexpr (ACCUM) {
#pragma unroll
            for (int t = 0; t < NTOUCH; ++t) asm volatile("" : : "v"(touched[t]));     // the touches end here
        }
        if (!nothing_to_add) {
            // C is reached through a descriptor over the wavefront's block (rows beyond the tile's end lie beyond its size;
            // a lane whose columns lie beyond N uses an offset beyond every size): loads return zeros there and stores
            // are dropped, so the epilogue has no branches and its loads can be issued ahead of the staging.
            uint8_t* stg = smem + kStage + wave * (kStage / 4);
            if constexpr (!ACCUM) rs_c = c_block_rsrc(cur);
            const int col_w = cur.n0 + wn * 128;
            if constexpr (OUT == OUT_STORE_BF16 || OUT == OUT_ACCUM_BF16) {
                // a lane's piece: eight columns (16 bytes of C) of row lane / 16 of every group of four rows
                const uint32_t c_lane = col_w + 8 * (lane & 15) < p.N ? (lane >> 4) * static_cast<uint32_t>(p.ldc) * 2u + (lane & 15) * 16u : kOutside;
                const uint32_t c_rows4 = 4u * static_cast<uint32_t>(p.ldc) * 2u;
                if constexpr (OUT == OUT_STORE_BF16) {
                    constexpr int PB = 128 * 2 + 16;                    // staged row: 128 bf16 + pad (sixteen rows x two quads of a write: 64 banks)
                    static_assert(64 * PB <= kStage / 4, "two passes of 64 rows");
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
#pragma unroll
                        for (int ii = 0; ii < 4; ++ii)
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                const v4f a = acc[j][4 * half + ii];
                                *reinterpret_cast<uint2*>(stg + (16 * ii + r16) * PB + (16 * j + 4 * kg) * 2) =
                                    make_uint2(pack_bf16x2_hw(acc_read(a[0]), acc_read(a[1])), pack_bf16x2_hw(acc_read(a[2]), acc_read(a[3])));
                            }
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const u32x4 v = *reinterpret_cast<const u32x4*>(stg + ((lane >> 4) + 4 * t) * PB + (lane & 15) * 16);
                            __builtin_amdgcn_raw_buffer_store_b128(v, rs_c, static_cast<int>(c_lane + (16 * half + t) * c_rows4), 0, 0);
                        }
                    }
                } else {
                    // fp32 sum of the old value and the product, one rounding (cublasGemmEx with a bf16 C, beta = 1)
                    constexpr int PF = 128 * 4 + 16;                    // staged row: 128 fp32 + pad (the sixteen rows of a quad column: 64 banks)
                    static_assert(32 * PF <= kStage / 4, "four passes of 32 rows");
                    // the next pass's rows of C are requested before this pass's are added to and stored
                    u32x4 c[8], c_ahead[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) c_ahead[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_c, static_cast<int>(c_lane + t * c_rows4), 0, 0);
#pragma unroll
                    for (int pass = 0; pass < 4; ++pass) {
#pragma unroll
                        for (int t = 0; t < 8; ++t) c[t] = c_ahead[t];
                        if (pass < 3) {
#pragma unroll
                            for (int t = 0; t < 8; ++t) c_ahead[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_c, static_cast<int>(c_lane + (8 * (pass + 1) + t) * c_rows4), 0, 0);
                        }
#pragma unroll
                        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                const v4f a = acc[j][2 * pass + ii];
                                *reinterpret_cast<float4*>(stg + (16 * ii + r16) * PF + (16 * j + 4 * kg) * 4) =
                                    make_float4(acc_read(a[0]), acc_read(a[1]), acc_read(a[2]), acc_read(a[3]));
                            }
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            const uint8_t* src = stg + ((lane >> 4) + 4 * t) * PF + (lane & 15) * 32;
                            const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 16);
                            u32x4 v;
                            v.x = pack_bf16x2_hw(lo.x + bf16_lo(c[t].x), lo.y + bf16_hi(c[t].x));
                            v.y = pack_bf16x2_hw(lo.z + bf16_lo(c[t].y), lo.w + bf16_hi(c[t].y));
                            v.z = pack_bf16x2_hw(hi.x + bf16_lo(c[t].z), hi.y + bf16_hi(c[t].z));
                            v.w = pack_bf16x2_hw(hi.z + bf16_lo(c[t].w), hi.w + bf16_hi(c[t].w));
                            __builtin_amdgcn_raw_buffer_store_b128(v, rs_c, static_cast<int>(c_lane + (8 * pass + t) * c_rows4), 0, 0);
                        }
                    }
                }
            } else {
                // fp32 C.  A lane's piece: four columns (16 bytes) of row lane / 32 of every pair of rows
                constexpr int PF = 128 * 4 + 16;
                static_assert(32 * PF <= kStage / 4, "four passes of 32 rows");
                const uint32_t c_lane = col_w + 4 * (lane & 31) < p.N ? (lane >> 5) * static_cast<uint32_t>(p.ldc) * 4u + (lane & 31) * 16u : kOutside;
                const uint32_t c_rows2 = 2u * static_cast<uint32_t>(p.ldc) * 4u;
                // ACCUM: C is read in groups of eight row pairs, a group ahead of the adds and stores
                [[maybe_unused]] u32x4 c[8], c_ahead[8];
                if constexpr (OUT == OUT_ACCUM_F32) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) c_ahead[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_c, static_cast<int>(c_lane + t * c_rows2), 0, 0);
                }
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
#pragma unroll
                    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const v4f a = acc[j][2 * pass + ii];
                            *reinterpret_cast<float4*>(stg + (16 * ii + r16) * PF + (16 * j + 4 * kg) * 4) =
                                make_float4(acc_read(a[0]), acc_read(a[1]), acc_read(a[2]), acc_read(a[3]));
                        }
#pragma unroll
                    for (int hg = 0; hg < 2; ++hg) {
                        if constexpr (OUT == OUT_ACCUM_F32) {
#pragma unroll
                            for (int t = 0; t < 8; ++t) c[t] = c_ahead[t];
                            if (2 * pass + hg < 7) {
#pragma unroll
                                for (int t = 0; t < 8; ++t)
                                    c_ahead[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_c, static_cast<int>(c_lane + (8 * (2 * pass + hg + 1) + t) * c_rows2), 0, 0);
                            }
                        }
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            const int tt = 8 * hg + t;
                            float4 v = *reinterpret_cast<const float4*>(stg + ((lane >> 5) + 2 * tt) * PF + (lane & 31) * 16);
                            if constexpr (OUT == OUT_ACCUM_F32) {
                                v.x += __uint_as_float(c[t].x); v.y += __uint_as_float(c[t].y); v.z += __uint_as_float(c[t].z); v.w += __uint_as_float(c[t].w);
                            }
                            u32x4 o;
                            o.x = __float_as_uint(v.x); o.y = __float_as_uint(v.y); o.z = __float_as_uint(v.z); o.w = __float_as_uint(v.w);
                            __builtin_amdgcn_raw_buffer_store_b128(o, rs_c, static_cast<int>(c_lane + (16 * pass + tt) * c_rows2), 0, 0);
                        }
                    }
                }
            }
        }
        __syncthreads();
        // the next tile: the one the fetch is in, or the one it has just left
        cur = tiles_ahead == 1 ? L : L_before;
        --tiles_ahead;
        if (!cur.valid) break;
        clear_acc();
    }
}

// one workgroup per CU, a multiple of 8 of them (launch position % 8 is the XCD), and no more than there are tiles
dim3 persistent_grid(long long tiles) {
    static const int cus = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 8) return 256;
        return v - v % 8;
    }();
    const long long want = 8 * ((tiles + 7) / 8);
    return dim3(static_cast<unsigned>(want < cus ? want : cus));
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
    // (the epilogue addresses a wavefront's 128 rows of C by 32-bit byte offsets from the block's first element)
    return aligned16(A) && aligned16(B) && lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 && ldc < (1 << 21) &&
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
    auto grid_for = [&](int row_tiles) { return persistent_grid(static_cast<long long>(row_tiles) * p.tiles_n); };
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
        return launch<true, OUT, true>(p, persistent_grid(blocks), st);
    }
    return launch<true, OUT, false>(p, persistent_grid(tiles), st);
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
    const dim3 grid = persistent_grid(total);
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
