// fp8_gemm, prefill kernel for gfx950 (reference: inference/kernel.py:118-172).
//
//   c[m,n] = sum_kb ( sum_{t<128} a[m,128kb+t] * b[n,128kb+t] ) * a_s[m,kb] * b_s[n/128,kb]
//
// 256 x 256 tile of C per workgroup, 8 wavefronts (4 along m x 2 along n), each
// owning 64 (m) x 128 (n) as 4 x 8 MFMA tiles of 16x16 with
// v_mfma_f32_16x16x128_f8f6f4: one instruction = one 128-wide scale block of K.
// The raw block dot products are folded into binary32 accumulators held in
// VGPRs with one FMA each by the block's scale.  The MFMA is issued with the
// weight rows (n) as its A operand and the activation rows (m) as its B
// operand, so a lane's four results share one m: the scale is a single value
// per lane and 16-row sub-tile, and the four results are consecutive in n.
//
// K blocks of A and B (both K-contiguous, 128 bytes per row) are copied
// global -> LDS with global_load_lds_dwordx4 (no VGPR staging), double
// buffered.  Such a load writes a wavefront's 64 x 16 bytes to consecutive LDS
// addresses, so the layout is chosen on the global side: 8 lanes fetch the 8
// 16-byte chunks of one row in a permuted order p = c ^ f(row), which leaves the
// later ds_read_b128 fragment reads (16 consecutive rows, same chunk) free of
// bank conflicts.
#include <cstdlib>
#include <type_traits>
#include "common.hpp"

namespace dsv3 {
namespace prefill {

constexpr int BN = 256;
constexpr int WAVES_M = 4, WAVES_N = 2;
constexpr int WN = BN / WAVES_N, SN = WN / 16;           // 128 columns = 8 MFMA tiles per wavefront
constexpr int THREADS = WAVES_M * WAVES_N * kWave;       // 512
constexpr int SC_STAGE = 8 * 256;                        // scales of one K block: one 64-float slot per wavefront

// Tile height TM and number of LDS stages S.  <256, 2>: the large-M shape, 64 x 128 per wavefront, 2 x 64 KiB of
// tiles.  <128, 3>: 32 x 128 per wavefront, 3 x 48 KiB -- the loads of a K block then have two blocks of time to
// land, which is what matters when a tile has little arithmetic per block (the ~128-row groups of an MoE layer:
// a global -> LDS round trip under load, ~1.4 us, is longer than such a block's MFMA time).
template <int TM, int S, int SB = S> struct Cfg {                    // S: activation (A) stages, SB: weight (B) stages
    static constexpr int WM = TM / WAVES_M, SM = WM / 16;
    static constexpr int A_LOADS = TM / 64, B_LOADS = BN / 64;        // 1 KiB wavefront-loads per wavefront and stage
    static constexpr int LOADS = A_LOADS + B_LOADS + 1;               // ... plus the scale load
    static constexpr int A_STAGE = TM * 128, B_STAGE = BN * 128;      // bytes per K block
    static constexpr int SS = SB > S ? SB : S;                        // scale slots
    static constexpr int LDS_A = 0, LDS_B = S * A_STAGE;              // [A stages | B stages | scale slots]
    static constexpr int LDS_SC = S * A_STAGE + SB * B_STAGE;
    static constexpr int LDS_BYTES = LDS_SC + SS * SC_STAGE;
    // grouped mode with scale batches (SCB) keeps, in place of the slots, two buffers of the scales of four K blocks --
    // 16 bytes per tile row, then the 64 x 16 bytes that wavefront 4 copies (lanes 0 and 1: b_s) -- and 1 KiB that
    // takes the copies nobody reads
    static constexpr int SCB_BUF = TM * 16 + 1024, LDS_DUMP = LDS_SC + 2 * SCB_BUF, LDS_BYTES_SCB = LDS_DUMP + 1024;
    static_assert(LDS_BYTES <= 160 * 1024 && LDS_BYTES_SCB <= 160 * 1024, "LDS of a gfx950 compute unit");
    static_assert(SB >= S, "the weights are the operand that comes from HBM");
};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// chunk permutation inside a 128-byte LDS row (see file comment)
// measured on gfx950 (SQ_LDS_BANK_CONFLICT == 0): 16 consecutive lanes reading the same logical chunk of
// 16 consecutive 128-byte rows do not collide when the chunk index is xor-ed with (row & 7) ^ (row >> 3 & 1)
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Workgroup barrier without the memory fence of __syncthreads(): that fence waits for every outstanding vector
// memory operation of the wavefront, i.e. also for the direct-to-LDS loads of later K blocks that are meant to stay
// in flight across the barrier.  What a barrier has to order here is spelled out at each use: the wavefront's own
// LDS reads (lgkmcnt) and exactly those of its loads whose data the other wavefronts are about to read (vmcnt(n)).
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    v8i r = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
    return r;
}

// Grouped mode (G): the rows of a (and of c) are cut into groups, each multiplied by its own weight matrix --
// the per-expert token lists of the reference's MoE layer (inference/model.py:684-689).  A row tile belongs to one
// group; a table built on the device (no host round trip for the group sizes) gives each tile slot its group,
// its first row in c and its row count, or group -1 for an unused slot.  a_rows, when given, maps a row of c to
// the row of a it reads (token gather); otherwise a and c share row numbers.
struct GroupTable {
    const int* tile_group;   // [tiles_m]
    const int* tile_row0;    // [tiles_m] first row of the tile in c (and in a_rows)
    const int* tile_rows;    // [tiles_m] 1 .. TM
    const int* a_rows;       // [rows of c] or nullptr
    int64_t b_stride;        // bytes between consecutive groups' weights
    int64_t bs_stride;       // floats between consecutive groups' weight scales
    // SwiGLU mode (SG): the tile's results do not leave as c but as act_quant(silu(h1) * h3), see swiglu_store
    uint8_t* sg_y;           // [rows of c, N / 2] e4m3
    float* sg_s;             // [rows of c, N / 256] scales
    int sg_ue8m0;            // scale format of the re-quantisation
};

// SwiGLU mode of the grouped kernels (inference/model.py:633 feeding the Linear of :631 -> inference/kernel.py:23-35):
// a group's weight is w1 stacked over w3 ([2 * inter, K]); a column tile takes the matching 128 rows of both as its
// two column halves -- rows tn * 128 .. + 127 of w1 for the first m-wavefront column, the same rows of w3 for the
// second -- so that after the K loop wavefront (wm, 0) holds h1 and wavefront (wm, 1) h3 of the same 64 x 128 outputs.
// Weight row behind row r (0 .. 255) of column tile tn, and the scale row of a column half:
__device__ __forceinline__ int sg_weight_row(int r, int tn, int inter) { return (r < 128 ? 0 : inter - 128) + tn * 128 + r; }
__device__ __forceinline__ int sg_scale_row(int half, int tn, int inter) { return (half ? inter / 128 : 0) + tn; }

// Epilogue of SwiGLU mode.  h3 crosses from wavefront (wm, 1) to (wm, 0) through LDS in the accumulators' own
// layout (lane l of the one writes what lane l of the other reads: 512 contiguous bytes per 16 x 16 tile, no bank
// conflicts); the first wavefront then forms g = bf16(bf16(silu(bf16 h1)) * bf16 h3) with the arithmetic of
// dsv3_swiglu_quant, reduces the row maximum over its 32 values and the three other lanes that hold the row, and
// writes 128 e4m3 bytes and one scale per row: the 128 columns of a tile are exactly one quantisation block.
// The result is what dsv3_fp8_gemm_grouped followed by dsv3_swiglu_quant produces, bit for bit; it saves that launch
// and three quarters of the bytes the GEMM writes.  acc[i][j]: column sub-tile i (16 columns), row sub-tile j.
template <int SM, typename SubRow>
__device__ __forceinline__ void swiglu_store(v4f (&acc)[8][SM], uint8_t* lds, int wm, int wn, int lane, SubRow sub_row,
                                             int m0, int rows_here, int tn, int inter, const GroupTable& g) {
    const int fr = lane & 15, fq = lane >> 4;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // every wavefront is done with the LDS stages
    v2u* xch = (v2u*)(lds + wm * (SM * 8 * 512));
    if (wn == 1) {
#pragma unroll
        for (int j = 0; j < SM; ++j)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                xch[(j * 8 + i) * 64 + lane] = v2u{ pack_bf16(acc[i][j][0], acc[i][j][1]), pack_bf16(acc[i][j][2], acc[i][j][3]) };
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (wn == 1) return;
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        if (sub_row(j) >= rows_here) continue;                         // (uniform) a sub-tile of padding rows
        float x1[8][4], big = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) { x1[i][e] = round_bf16(acc[i][j][e]); big = fmaxf(big, fabsf(x1[i][e])); }
        float gv[8][4];
        const bool fast = __all(big < 64.f);                            // (false for NaN as well)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const v2u h3 = xch[(j * 8 + i) * 64 + lane];
            const float x3[4] = { bf16lo_to_f32(h3[0]), bf16hi_to_f32(h3[0]), bf16lo_to_f32(h3[1]), bf16hi_to_f32(h3[1]) };
#pragma unroll
            for (int e = 0; e < 4; ++e) gv[i][e] = fast ? swiglu_bf16<true>(x1[i][e], x3[e]) : swiglu_bf16<false>(x1[i][e], x3[e]);
        }
        uint32_t abits = 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) abits = umax_u32(abits, abs_bits(gv[i][e]));
        abits = umax_u32(abits, (uint32_t)__shfl_xor((int)abits, 16));  // the row's other three lanes
        abits = umax_u32(abits, (uint32_t)__shfl_xor((int)abits, 32));
        const float sc = block_scale(abits, g.sg_ue8m0 != 0);
        const bool finite = __all(block_is_finite(abits));              // uniform, so that only one quotient is evaluated
        const float rcp = 1.0f / sc;
        // the sub-tile's 16 rows x 128 bytes pass through the part of the exchange area this wavefront has just read
        // (16-byte chunks xor-ed with the row), so that a store instruction writes 8 whole rows instead of 16-byte pieces
        uint8_t* stg = (uint8_t*)(xch + j * 8 * 64);
        auto quantise = [&](auto fast_tag) {
            constexpr bool FAST = decltype(fast_tag)::value;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float q[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) q[e] = block_quotient(gv[i][e], sc, rcp, FAST);
                *(uint32_t*)(stg + fr * 128 + ((i ^ (fr & 7)) * 16) + fq * 4) = pack_fp8x4(q[0], q[1], q[2], q[3]);
            }
        };
        if (finite) quantise(std::true_type{}); else quantise(std::false_type{});
        const int r0 = sub_row(j);
        if (fq == 0 && r0 + fr < rows_here) g.sg_s[(size_t)(m0 + r0 + fr) * (size_t)(inter / 128) + tn] = sc;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int rr = p * 8 + (lane >> 3), ch = lane & 7;
            const v4u v = *(const v4u*)(stg + rr * 128 + ((ch ^ (rr & 7)) * 16));
            if (r0 + rr < rows_here)
                *(v4u*)(g.sg_y + (size_t)(m0 + r0 + rr) * (size_t)inter + tn * 128 + ch * 16) = v;
        }
    }
}

// One workgroup's tile (grouped mode: tile slot) from start to end; the kernels below are thin wrappers.
// P2: every scale is a power of two (act_quant's ue8m0 format and checkpoints whose block scales are stored that
// way).  The block scales then ride in the MFMA's E8M0 scale operands and the products of all K blocks accumulate
// inside the matrix core: no fold, no vector-ALU work in the K loop.
// SCB (grouped mode; K a multiple of 512, a_s and b_s 16-byte aligned): the scales are copied four K blocks at a time,
// see issue_scales.
template <int CD, bool G, int TM, int S, int SB = S, bool P2 = false, bool SG = false, bool SCB = false>
__device__ __forceinline__ void prefill_tile(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c,
        int M, int N, int K, int tiles_m, int tiles_n, int tn_first, int kb_per_split, int ldc, GroupTable g,
        int wg) {                           // index of the workgroup among those that run this configuration
    using C = Cfg<TM, S, SB>;
    constexpr int SS = C::SS;
    constexpr int WM = C::WM, SM = C::SM, A_LOADS = C::A_LOADS, B_LOADS = C::B_LOADS;
    constexpr int A_STAGE = C::A_STAGE, B_STAGE = C::B_STAGE, LDS_A = C::LDS_A, LDS_B = C::LDS_B, LDS_SC = C::LDS_SC;
    static_assert(!SG || (G && !P2 && CD == DSV3_BF16), "SwiGLU mode: grouped, binary32 scales, bf16 intermediate");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    // ---- workgroup -> tile.  Consecutive workgroup ids go to consecutive XCDs (8 of them, each with its own L2).
    // Dense mode gives every XCD a contiguous run of tiles and walks it in bands of GROUP_M tile rows.  Grouped
    // mode deals the row tiles round-robin over the XCDs -- the live ones sit at the front of the tile table, and a
    // contiguous split would leave the XCDs that get the unused tail idle -- and keeps the column tiles of a row
    // tile on one XCD (they share the gathered rows of a).
    int m0, n0, rows_here;              // first row of the tile in c, first column, valid rows
    int tn_idx = 0;                     // (SwiGLU mode: the column tile)
    if (G) {
        const int x = wg % 8, idx = wg / 8;
        const int tm = (idx / tiles_n) * 8 + x, tn = idx - (idx / tiles_n) * tiles_n;
        if (tm >= tiles_m) return;      // uniform over the workgroup, before any barrier
        const int grp = g.tile_group[tm];
        if (grp < 0) return;
        m0 = g.tile_row0[tm];
        rows_here = g.tile_rows[tm];
        n0 = (tn_first + tn) * BN;
        tn_idx = tn_first + tn;
        b += (size_t)grp * g.b_stride;
        b_s += (size_t)grp * g.bs_stride;
    } else {
        const int T = tiles_m * tiles_n;
        int pid = wg;
        {
            const int q = T / 8, r = T % 8, x = pid % 8;
            pid = x * q + (x < r ? x : r) + pid / 8;
        }
        constexpr int GROUP_M = 4;
        const int band = pid / (GROUP_M * tiles_n);
        const int band_rows = min(GROUP_M, tiles_m - band * GROUP_M);
        const int in_band = pid - band * GROUP_M * tiles_n;
        const int tm = band * GROUP_M + in_band % band_rows;
        const int tn = in_band / band_rows;
        m0 = tm * TM; n0 = (tn_first + tn) * BN;
        rows_here = min(TM, M - m0);
    }
    // row of a behind row r of the tile; rows past the tile's end repeat its last row (their results are dropped)
    auto a_row = [&](int r) -> uint32_t {
        const int rr = m0 + min(r, rows_here - 1);
        return (uint32_t)((G && g.a_rows) ? g.a_rows[rr] : rr);
    };

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & (WAVES_M - 1), wn = wave / WAVES_M;
    // K blocks of this workgroup: all of them, or slice blockIdx.y of a split over K (dense mode only), whose
    // partial sums go to slab blockIdx.y of c
    const int KBT = K / 128;
    const int kb0 = blockIdx.y * kb_per_split;
    const int KB = min(kb_per_split, KBT - kb0);
    // c has row stride ldc and starts at column tn_first * BN (ldc = N, tn_first = 0 for a plain launch; a slab
    // of partial sums covers only the launch's column range)
    c += (size_t)blockIdx.y * (size_t)M * (size_t)ldc;
    const int n_base = ldc == N ? 0 : tn_first * BN;
    a += (size_t)kb0 * 128u; b += (size_t)kb0 * 128u;

    // ---- global -> LDS copy plan: a stage is TM rows of A, then 256 of B, in 1 KiB wavefront-loads of 8 rows;
    // wavefront w issues A loads t*8 + w (t < A_LOADS) and B loads t*8 + w (t < B_LOADS).
    // Lane l of a load -> row 8q + l/8, LDS chunk l%8, global chunk (l%8)^f(row).
    uint32_t src_off[A_LOADS + B_LOADS];
    // load t of K block kb into LDS stage `stage`: t < A_LOADS is the activation part, the rest the weight part
    auto issue_load = [&](int t, int kb, int stage) {
        const bool is_a = t < A_LOADS;
        const int q = (is_a ? t : t - A_LOADS) * 8 + wave;
        const uint8_t* base = is_a ? a : b;
        const int dst = (is_a ? LDS_A + stage * A_STAGE : LDS_B + stage * B_STAGE) + q * 1024;
        __builtin_amdgcn_global_load_lds((gptr_t)(base + src_off[t] + (uint32_t)kb * 128u),
                                         (lptr_t)(lds + dst), 16, 0, 0);
    };
    // The weight part of K block 0 is requested right here, ahead of everything that depends on the row map: a
    // group's weights come from HBM, the longest wait of the tile's start, and a gathered row number is itself a
    // dependent load.  The row numbers are requested first (older loads return first, so waiting for them does not
    // wait for the copies behind them), then the four weight copies, then the activation addresses are formed.
    uint32_t a_src_row[A_LOADS];
#pragma unroll
    for (int t = 0; t < A_LOADS; ++t) a_src_row[t] = a_row((t * 8 + wave) * 8 + (lane >> 3));
    const uint32_t a_scale_row = a_row(wave * 64 + lane);
#pragma unroll
    for (int t = A_LOADS; t < A_LOADS + B_LOADS; ++t) {
        const int row = ((t - A_LOADS) * 8 + wave) * 8 + (lane >> 3);
        src_off[t] = (uint32_t)(SG ? sg_weight_row(row, tn_idx, N / 2) : min(n0 + row, N - 1)) * (uint32_t)K + (((lane & 7) ^ swz(row)) * 16);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = A_LOADS; t < A_LOADS + B_LOADS; ++t) issue_load(t, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < A_LOADS; ++t) {
        const int row = (t * 8 + wave) * 8 + (lane >> 3);
        src_off[t] = a_src_row[t] * (uint32_t)K + (((lane & 7) ^ swz(row)) * 16);
    }

    // ---- fragment read addresses.  A lane reads row (lane&15) of a 16-row sub-tile and the 32 bytes
    // at K offset 32*(lane>>4), i.e. chunks 2*(lane>>4) and 2*(lane>>4)+1, permuted by f(row).
    const int fr = lane & 15, fq = lane >> 4;
    const int fx = swz(fr);                                   // sub-tile bases are multiples of 16 rows
    const int c0 = ((2 * fq) ^ fx) * 16, c1 = ((2 * fq + 1) ^ fx) * 16;
    // 16-row sub-tile j of this wavefront: consecutive rows in dense mode; in grouped mode the sub-tiles are
    // dealt round-robin over the four m-wavefronts, so that a tile with few valid rows (a small expert) leaves
    // every SIMD the same share of work instead of idling two of them
    auto sub_row = [&](int j) { return G ? (j * WAVES_M + wm) * 16 : wm * WM + j * 16; };
    constexpr int A_JSTRIDE = (G ? WAVES_M : 1) * 2048;       // LDS bytes between consecutive sub-tiles of a wavefront
    const int a_rd = LDS_A + (sub_row(0) + fr) * 128;         // + j*A_JSTRIDE + stage*A_STAGE
    const int b_rd = LDS_B + (wn * WN + fr) * 128;            // + i*16*128 + stage*B_STAGE

    // ---- scales.  They take the same route as the tiles: global -> LDS (4 bytes per lane), one slot per stage,
    // requested with the tiles, read back after the block's barrier.  An ordinary global load inside the K
    // loop is not an option: issued behind the wavefront's outstanding direct-to-LDS loads it holds the
    // wavefront until those have returned -- a memory round trip per K block, measured at 30% of the kernel.
    // Wavefronts 0-3 fetch a_s[row, kb] of 64 tile rows each (rows past the tile repeat its last row), lanes 0 and 1
    // of wavefront 4 the b_s rows of the two column halves; every other lane of wavefronts 4-7 repeats the first of
    // those addresses into slots nobody reads, which keeps the loop free of branches and costs one cache line per
    // instruction instead of 64.
    const int nb_last = (N - 1) / 128;
    const float* sc_base = wave < 4 ? a_s : b_s;
    const int b_scale_row = SG ? sg_scale_row(wave == 4 ? min(lane, 1) : 0, tn_idx, N / 2)
                               : min(n0 / 128 + (wave == 4 ? min(lane, 1) : 0), nb_last);
    const uint32_t sc_off = (wave < 4 ? a_scale_row * (uint32_t)KBT : (uint32_t)b_scale_row * (uint32_t)KBT) + (uint32_t)kb0;
    // SCB.  A group's weights stream from HBM, and there the lines of the activation scales -- one per row and K block,
    // 4 bytes used of each -- cost 6 % of a 128-row slot's time.  With SCB every wavefront copies 16 bytes per lane, the
    // scales of FOUR K blocks, into one of two buffers in the block that would have requested the first of them, and one
    // line that nobody reads (sc_one_line: a 16-byte aligned address every lane may read) in the other three, which
    // keeps the counted waits as they are.  No branch on the block number or the wavefront: the addresses are selected
    // (a branch in the middle of a block splits the region its instruction order is pinned in, and that costs spills).
    static_assert(!SCB || G, "scale batches: grouped mode");
    constexpr int SCB_BUF = C::SCB_BUF, LDS_DUMP = C::LDS_DUMP;
    const bool sc_live = wave < TM / 64 || wave == 4;
    const int sc_dst = LDS_SC + (wave < TM / 64 ? wave * 1024 : TM * 16);
    const uint32_t sc_one_line = (uint32_t)__builtin_amdgcn_readfirstlane((int)sc_off);
    auto issue_scales = [&](int kb, int stage) {
        if constexpr (SCB) {
            const bool real = sc_live && (kb & 3) == 0;
            __builtin_amdgcn_global_load_lds((gptr_t)(sc_base + (real ? sc_off + (uint32_t)kb : sc_one_line)),
                                             (lptr_t)(lds + (real ? sc_dst + ((kb >> 2) & 1) * SCB_BUF : LDS_DUMP)), 16, 0, 0);
        } else
            __builtin_amdgcn_global_load_lds((gptr_t)(sc_base + sc_off + (uint32_t)kb),
                                             (lptr_t)(lds + LDS_SC + stage * SC_STAGE + wave * 256), 4, 0, 0);
    };
    // the scales of K block kb (whose slot is `stage`): a_s of the lane's row of sub-tile j, b_s of the wavefront's columns
    auto lds_as = [&](int j, int stage, int kb) {
        if constexpr (SCB) return *(const float*)(lds + LDS_SC + ((kb >> 2) & 1) * SCB_BUF + (kb & 3) * 4 + (sub_row(j) + fr) * 16);
        else return *(const float*)(lds + LDS_SC + stage * SC_STAGE + (sub_row(j) + fr) * 4);
    };
    auto lds_bs = [&](int stage, int kb) {
        if constexpr (SCB) return *(const float*)(lds + LDS_SC + ((kb >> 2) & 1) * SCB_BUF + (kb & 3) * 4 + TM * 16 + wn * 16);
        else return *(const float*)(lds + LDS_SC + stage * SC_STAGE + (256 + wn) * 4);
    };

    v4f acc[SN][SM];
#pragma unroll
    for (int i = 0; i < SN; ++i)
#pragma unroll
        for (int j = 0; j < SM; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    // Software pipeline.  Per 16-column step i of a K block the wavefront issues
    //     ds_read x2 (weights of step i+2) | MFMA j=0 | FMA of the pending tile | MFMA 1 | FMA tile 0 | MFMA 2 |
    //     FMA tile 1 | MFMA 3 | FMA tile 2            (tile 3 stays pending into the next step)
    // so every FMA reads a result that was issued two MFMAs earlier and the matrix pipe never waits on the
    // vector pipe.
    //
    // The workgroup barrier of a K block sits before step kSync = SN-2, not at the block's end: by then every
    // fragment the block still needs is in registers, so after the barrier the block's LDS stage can be refilled
    // (block kb+S) and the first fragments of block kb+1 are read from the next stage while the last
    // 2 x SM MFMAs of block kb run.  The next block then starts with its operands already in registers.
    //
    // Loads are issued in program order and retire in order.  Per K block a wavefront issues, after barrier kb:
    // the activation part and the scales of block kb+S (steps kSync, kSync+1), then the weight part of block kb+S
    // (steps 0, 1 of block kb+1) -- spread out, because a burst of every wavefront's loads right after the barrier
    // stalls instruction issue.  At barrier kb the data of block kb+1 must be there; everything issued later
    // belongs to blocks kb+2 .. kb+S-1, so the wait is vmcnt((S-2) * loads per block).
    constexpr int kSync = SN - 2;
    // (with more weight stages than activation stages the weight part of a block is requested SB - S blocks
    // earlier: at barrier kb the loads that may still be in flight are the weight parts of blocks kb+2 .. kb+SB-1
    // and the activation parts and scales of blocks kb+2 .. kb+S-1, all of them younger than anything of block kb+1)
    constexpr int kInFlight = (SB - 2) * B_LOADS + (S - 2) * (A_LOADS + 1);
    constexpr int kWaitSync = 0x0f70 | kInFlight;
    static_assert(kInFlight < 16, "vmcnt immediate");
    auto next_a = [](int st) { return st + 1 == S ? 0 : st + 1; };
    auto next_b = [](int st) { return st + 1 == SB ? 0 : st + 1; };
    auto next_s = [](int st) { return st + 1 == SS ? 0 : st + 1; };
    auto prev_b = [](int st) { return st == 0 ? SB - 1 : st - 1; };
    // scale slot of block kb + S seen from the slot of block kb
    auto ahead_s = [](int st) { return (st + S) % SS; };
    // sub-tiles of this wavefront that hold at least one valid row (all of them in dense mode; the clamped rows of
    // an edge tile are computed and dropped there).  The pipeline below is instantiated per count, so a wavefront
    // issues MFMAs and FMAs only for live sub-tiles; one without any only feeds LDS and keeps the barriers.
    const int ja_live = G ? max(0, min(SM, ((rows_here + 15) / 16 - wm + WAVES_M - 1) / WAVES_M)) : SM;

#define DSV3_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
    auto pipeline = [&](auto ja_tag) {
        constexpr int JA = decltype(ja_tag)::value;
        // prologue: the rest of block 0 (its weight part is in flight already), then the blocks the steady state
        // expects to be in flight -- 1 .. S-2 completely and the activation part + scales of block S-1 -- and only
        // then the wait for block 0: everything requested after it may stay in flight across the barrier
#pragma unroll
        for (int t = 0; t < A_LOADS; ++t) issue_load(t, 0, 0);
        issue_scales(0, 0);
        constexpr int kLater = [] {
            int n = 0;
            for (int blk = 1; blk < SS; ++blk) n += (blk < S ? A_LOADS + 1 : 0) + (blk < SB - 1 ? B_LOADS : 0);
            return n;
        }();
        static_assert(kLater < 16, "vmcnt immediate");
#pragma unroll
        for (int blk = 1; blk < SS; ++blk) {
            if (blk < S) {
#pragma unroll
                for (int t = 0; t < A_LOADS; ++t) issue_load(t, min(blk, KB - 1), blk);
                issue_scales(min(blk, KB - 1), blk);
            }
            if (blk < SB - 1) {
#pragma unroll
                for (int t = A_LOADS; t < A_LOADS + B_LOADS; ++t) issue_load(t, min(blk, KB - 1), blk);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70 | kLater);
        wg_barrier();
        if constexpr (JA == 0) {
            int st_a = 0, st_b = 0, st_s = 0;
            for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
                for (int t = A_LOADS; t < A_LOADS + B_LOADS; ++t) issue_load(t, min(kb - 1 + SB, KB - 1), prev_b(st_b));
                __builtin_amdgcn_s_waitcnt(kWaitSync);
                wg_barrier();
#pragma unroll
                for (int t = 0; t < A_LOADS; ++t) issue_load(t, min(kb + S, KB - 1), st_a);
                issue_scales(min(kb + S, KB - 1), ahead_s(st_s));
                st_a = next_a(st_a); st_b = next_b(st_b); st_s = next_s(st_s);
            }
            __builtin_amdgcn_s_waitcnt(0x0f70);
        } else if constexpr (P2) {
        // biased exponents (E8M0) of the block's scales: the weights' (MFMA A operand, one value per wavefront) and
        // the activations' (B operand, the lane's row)
        int eb, ea[JA], eb_nxt, ea_nxt[JA];
        auto e8m0 = [](float x) { return (int)(f32_as_u32(x) >> 23); };
        eb_nxt = e8m0(lds_bs(0, 0));
#pragma unroll
        for (int j = 0; j < JA; ++j) ea_nxt[j] = e8m0(lds_as(j, 0, 0));
        v8i nf0, nf1, mf[JA];
        {
            const uint8_t* as_base = lds + a_rd;
            const uint8_t* bs_base = lds + b_rd;
            nf0 = join(*(const v4i*)(bs_base + c0), *(const v4i*)(bs_base + c1));
#pragma unroll
            for (int j = 0; j < JA; ++j)
                mf[j] = join(*(const v4i*)(as_base + j * A_JSTRIDE + c0), *(const v4i*)(as_base + j * A_JSTRIDE + c1));
            nf1 = join(*(const v4i*)(bs_base + 2048 + c0), *(const v4i*)(bs_base + 2048 + c1));
        }
        int st_a = 0, st_b = 0, st_s = 0;
        for (int kb = 0; kb < KB; ++kb) {
            const int sa_next = next_a(st_a), sb_next = next_b(st_b), ss_next = next_s(st_s);
            const uint8_t* bs_base = lds + b_rd + st_b * B_STAGE;
            const uint8_t* as_next = lds + a_rd + sa_next * A_STAGE;
            const uint8_t* bs_next = lds + b_rd + sb_next * B_STAGE;
            const int kb_w = min(kb - 1 + SB, KB - 1), kb_a = min(kb + S, KB - 1);
            eb = eb_nxt;
#pragma unroll
            for (int j = 0; j < JA; ++j) ea[j] = ea_nxt[j];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < SN; ++i) {
                if (i == kSync) {
                    __builtin_amdgcn_s_waitcnt(kWaitSync);
                    wg_barrier();
                    eb_nxt = e8m0(lds_bs(ss_next, kb + 1));
#pragma unroll
                    for (int j = 0; j < JA; ++j) ea_nxt[j] = e8m0(lds_as(j, ss_next, kb + 1));
                    issue_scales(kb_a, ahead_s(st_s));
                    __builtin_amdgcn_sched_barrier(0);
                }
                v8i nf2;
                if (i < kSync)
                    nf2 = join(*(const v4i*)(bs_base + (i + 2) * 2048 + c0), *(const v4i*)(bs_base + (i + 2) * 2048 + c1));
                else
                    nf2 = join(*(const v4i*)(bs_next + (i - kSync) * 2048 + c0), *(const v4i*)(bs_next + (i - kSync) * 2048 + c1));
#pragma unroll
                for (int j = 0; j < JA; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(nf0, mf[j], acc[i][j], 0, 0, 0, eb, 0, ea[j]);
                    if (i == SN - 1) mf[j] = join(*(const v4i*)(as_next + j * A_JSTRIDE + c0), *(const v4i*)(as_next + j * A_JSTRIDE + c1));
                }
                if (i >= kSync) {
                    constexpr int kHalf = (A_LOADS + 1) / 2;
#pragma unroll
                    for (int t = (i == kSync ? 0 : kHalf); t < (i == kSync ? kHalf : A_LOADS); ++t) issue_load(t, kb_a, st_a);
                }
                if (i < 2) {
#pragma unroll
                    for (int t = 0; t < B_LOADS / 2; ++t) issue_load(A_LOADS + i * (B_LOADS / 2) + t, kb_w, prev_b(st_b));
                }
                nf0 = nf1;
                nf1 = nf2;
                DSV3_SGB(0x100, 2);
#pragma unroll
                for (int j = 0; j < JA; ++j) {
                    DSV3_SGB(0x008, 1);
                    if (i == SN - 1) DSV3_SGB(0x100, 2);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            st_a = sa_next; st_b = sb_next; st_s = ss_next;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        } else {
        float sc[JA], sc_nxt[JA];
        {
            const float bs = lds_bs(0, 0);
#pragma unroll
            for (int j = 0; j < JA; ++j) sc_nxt[j] = lds_as(j, 0, 0) * bs;
#pragma unroll
            for (int j = 0; j < JA; ++j) sc[j] = 0.f;
        }
        v4f pend = {0.f, 0.f, 0.f, 0.f};      // raw dot products of (i = SN-1, j = JA-1) of the previous K block
        v8i nf0, nf1, mf[JA];                 // weight fragments of steps i, i+1 (MFMA A operand); activation fragments (B operand)
        {
            const uint8_t* as_base = lds + a_rd;
            const uint8_t* bs_base = lds + b_rd;
            nf0 = join(*(const v4i*)(bs_base + c0), *(const v4i*)(bs_base + c1));
#pragma unroll
            for (int j = 0; j < JA; ++j)
                mf[j] = join(*(const v4i*)(as_base + j * A_JSTRIDE + c0), *(const v4i*)(as_base + j * A_JSTRIDE + c1));
            nf1 = join(*(const v4i*)(bs_base + 2048 + c0), *(const v4i*)(bs_base + 2048 + c1));
        }

        int st_a = 0, st_b = 0, st_s = 0;     // LDS stages of block kb: activations, weights, scales
        for (int kb = 0; kb < KB; ++kb) {
            const int sa_next = next_a(st_a), sb_next = next_b(st_b), ss_next = next_s(st_s);
            const uint8_t* bs_base = lds + b_rd + st_b * B_STAGE;
            const uint8_t* as_next = lds + a_rd + sa_next * A_STAGE;
            const uint8_t* bs_next = lds + b_rd + sb_next * B_STAGE;

            // branch-free: past the end the loop re-fetches the last block into stages nobody reads again
            const int kb_w = min(kb - 1 + SB, KB - 1), kb_a = min(kb + S, KB - 1);

            // fold the tile left over from the previous K block with that block's scale, then switch scales
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[SN - 1][JA - 1][e] = __builtin_fmaf(pend[e], sc[JA - 1], acc[SN - 1][JA - 1][e]);
#pragma unroll
            for (int j = 0; j < JA; ++j) sc[j] = sc_nxt[j];
            __builtin_amdgcn_sched_barrier(0);

#pragma unroll
            for (int i = 0; i < SN; ++i) {
                if (i == kSync) {
                    // every LDS read of this stage has returned and this wavefront's share of the next stage
                    // (tiles and scales of block kb+1) has landed
                    __builtin_amdgcn_s_waitcnt(kWaitSync);
                    wg_barrier();
                    {
                        const float bs = lds_bs(ss_next, kb + 1);
#pragma unroll
                        for (int j = 0; j < JA; ++j) sc_nxt[j] = lds_as(j, ss_next, kb + 1) * bs;
                    }
                    issue_scales(kb_a, ahead_s(st_s));
                    __builtin_amdgcn_sched_barrier(0);
                }
                // weight rows are streamed two steps ahead; the last two steps fetch steps 0 and 1 of the next block
                v8i nf2;
                if (i < kSync)
                    nf2 = join(*(const v4i*)(bs_base + (i + 2) * 2048 + c0), *(const v4i*)(bs_base + (i + 2) * 2048 + c1));
                else
                    nf2 = join(*(const v4i*)(bs_next + (i - kSync) * 2048 + c0), *(const v4i*)(bs_next + (i - kSync) * 2048 + c1));
                const v4f z = {0.f, 0.f, 0.f, 0.f};
                v4f p[JA];
                p[0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(nf0, mf[0], z, 0, 0, 0, 0, 0, 0);
                if (i == SN - 1) mf[0] = join(*(const v4i*)(as_next + c0), *(const v4i*)(as_next + c1));
                if (i > 0) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i - 1][JA - 1][e] = __builtin_fmaf(pend[e], sc[JA - 1], acc[i - 1][JA - 1][e]);
                }
#pragma unroll
                for (int j = 1; j < JA; ++j) {
                    p[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(nf0, mf[j], z, 0, 0, 0, 0, 0, 0);
                    if (i == SN - 1) mf[j] = join(*(const v4i*)(as_next + j * A_JSTRIDE + c0), *(const v4i*)(as_next + j * A_JSTRIDE + c1));
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j - 1][e] = __builtin_fmaf(p[j - 1][e], sc[j - 1], acc[i][j - 1][e]);
                }
                // refill, see above: activation part of block kb+S after the barrier, weight part of block kb-1+S
                // at the start of the block
                if (i >= kSync) {                           // first half (rounded up) at step kSync, the rest at kSync + 1
                    constexpr int kHalf = (A_LOADS + 1) / 2;
#pragma unroll
                    for (int t = (i == kSync ? 0 : kHalf); t < (i == kSync ? kHalf : A_LOADS); ++t) issue_load(t, kb_a, st_a);
                }
                if (i < 2) {
#pragma unroll
                    for (int t = 0; t < B_LOADS / 2; ++t) issue_load(A_LOADS + i * (B_LOADS / 2) + t, kb_w, prev_b(st_b));
                }
                pend = p[JA - 1];
                nf0 = nf1;
                nf1 = nf2;
                DSV3_SGB(0x100, 2);
                DSV3_SGB(0x008, 1);
                if (i == SN - 1) DSV3_SGB(0x100, 2);
                if (i > 0) DSV3_SGB(0x002, 4);
#pragma unroll
                for (int j = 1; j < JA; ++j) {
                    DSV3_SGB(0x008, 1);
                    if (i == SN - 1) DSV3_SGB(0x100, 2);
                    DSV3_SGB(0x002, 4);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            st_a = sa_next; st_b = sb_next; st_s = ss_next;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[SN - 1][JA - 1][e] = __builtin_fmaf(pend[e], sc[JA - 1], acc[SN - 1][JA - 1][e]);
        __builtin_amdgcn_s_waitcnt(0x0f70);             // the clamped refills of the last blocks are still in flight
        }
    };
    // 16-bit outputs with full-width rows are stored through LDS (see the epilogue)
    const bool lds_epilogue = CD != DSV3_F32 && (N % 8) == 0 && ldc == N;
    const bool f32_lds_epilogue = CD == DSV3_F32 && (N % 4) == 0 && (ldc % 4) == 0 && (SN % 2) == 0;
    static_assert(SM >= 2 && SM <= 4, "dispatch below");
    if (!G || ja_live == SM) pipeline(std::integral_constant<int, SM>{});
    else if (SM >= 4 && ja_live == 3) pipeline(std::integral_constant<int, (SM >= 4 ? 3 : 1)>{});
    else if (SM >= 3 && ja_live == 2) pipeline(std::integral_constant<int, (SM >= 3 ? 2 : 1)>{});
    else if (ja_live == 1)  pipeline(std::integral_constant<int, 1>{});
    else {
        pipeline(std::integral_constant<int, 0>{});
        if (SG) { wg_barrier(); wg_barrier(); return; }         // the two barriers of swiglu_store
        if (lds_epilogue || f32_lds_epilogue) wg_barrier();     // the barrier the other wavefronts take before they reuse the LDS stages
        return;
    }
#undef DSV3_SGB
    if constexpr (SG) {
        static_assert(SN == 8, "swiglu_store: eight column sub-tiles per wavefront");
        swiglu_store<SM>(acc, lds, wm, wn, lane, sub_row, m0, rows_here, tn_idx, N / 2, g);
        return;
    }

    // ---- epilogue: lane holds c[m][n .. n+3] for every (i, j)
    const bool vec_ok = (N % 4) == 0 && (ldc % 4) == 0;
    if (lds_epilogue) {
        // 16-bit outputs go through LDS (free now: one barrier, then a private 256-byte-per-row region per
        // wavefront) so that a store instruction writes 4 rows x 256 contiguous bytes instead of 16 rows x four
        // 8-byte pieces.  16-byte chunks are xor-ed with the row, which spreads both the 8-byte writes of the 16 rows
        // of a sub-tile and the 16-byte reads of a row over all banks.
        wg_barrier();
        uint8_t* stg = lds + wave * (WM * 256);
#pragma unroll
        for (int j = 0; j < SM; ++j)
#pragma unroll
            for (int i = 0; i < SN; ++i) {
                v2u o;
                if (CD == DSV3_BF16) o = v2u{ pack_bf16(acc[i][j][0], acc[i][j][1]), pack_bf16(acc[i][j][2], acc[i][j][3]) };
                else o = v2u{ pack_f16(acc[i][j][0], acc[i][j][1]), pack_f16(acc[i][j][2], acc[i][j][3]) };
                const int lr = j * 16 + fr, chunk = (i * 2 + (fq >> 1)) ^ fr;
                *(v2u*)(stg + lr * 256 + chunk * 16 + (fq & 1) * 8) = o;
            }
        const int rr = lane >> 4, ch = lane & 15;
#pragma unroll
        for (int p = 0; p < WM / 4; ++p) {
            const int lr = p * 4 + rr;                                   // local row: sub-tile lr / 16, row lr % 16
            const v4u v = *(const v4u*)(stg + lr * 256 + ((ch ^ (lr & 15)) * 16));
            const int r = sub_row(lr >> 4) + (lr & 15);
            const int n = n0 + wn * WN + ch * 8;
            if (r < rows_here && n < N)                                   // N % 8 == 0: a chunk is inside or outside
                *(v4u*)(c + (size_t)(m0 + r) * N + n) = v;
        }
        return;
    }
    if (f32_lds_epilogue) {
        // The same for fp32 results (the slabs of a K slice, mostly), half of the wavefront's columns per pass so that
        // the region stays at 256 bytes per row: a store instruction then writes 4 rows x 256 contiguous bytes
        // instead of 16 rows x 64.
        wg_barrier();
        uint8_t* stg = lds + wave * (WM * 256);
        const int rr = lane >> 4, ch = lane & 15;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int j = 0; j < SM; ++j)
#pragma unroll
                for (int i = 0; i < SN / 2; ++i) {
                    const int lr = j * 16 + fr, chunk = (i * 4 + fq) ^ fr;
                    *(v4f*)(stg + lr * 256 + chunk * 16) = acc[h * (SN / 2) + i][j];
                }
#pragma unroll
            for (int p = 0; p < WM / 4; ++p) {
                const int lr = p * 4 + rr;
                const v4f v = *(const v4f*)(stg + lr * 256 + ((ch ^ (lr & 15)) * 16));
                const int r = sub_row(lr >> 4) + (lr & 15);
                const int n = n0 + wn * WN + h * (WN / 2) + ch * 4;
                if (r < rows_here && n < N)                               // N % 4 == 0: a chunk is inside or outside
                    *(v4f*)(c + (size_t)(m0 + r) * ldc + (n - n_base)) = v;
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        const int r = sub_row(j) + fr;
        if (r >= rows_here) continue;
        const int m = m0 + r;
#pragma unroll
        for (int i = 0; i < SN; ++i) {
            const int n = n0 + wn * WN + i * 16 + fq * 4;
            typename OutT<CD>::type* dst = c + (size_t)m * ldc + (n - n_base);
            if (vec_ok && n + 3 < N) {
                if (CD == DSV3_F32) {
                    *(v4f*)dst = acc[i][j];
                } else if (CD == DSV3_BF16) {
                    v2u o = { pack_bf16(acc[i][j][0], acc[i][j][1]), pack_bf16(acc[i][j][2], acc[i][j][3]) };
                    *(v2u*)dst = o;
                } else {
                    v2u o = { pack_f16(acc[i][j][0], acc[i][j][1]), pack_f16(acc[i][j][2], acc[i][j][3]) };
                    *(v2u*)dst = o;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) dst[e] = cvt_out<CD>(acc[i][j][e]);
            }
        }
    }
}

#include "fp8_gemm_pingpong.hpp"

inline bool use_pingpong() { static const bool v = getenv("DSV3_PREFILL_NOPP") == nullptr; return v; }
inline bool use_pingpong_short() { static const bool v = use_pingpong() && getenv("DSV3_PREFILL_NOPP128") == nullptr; return v; }

template <int CD, bool P2 = false, int SM = 4>
__global__ __launch_bounds__(THREADS, 1) void fp8_gemm_pingpong_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c,
        int M, int N, int K, int tiles_m, int tiles_n, int tn_first, int kb_per_split, int ldc) {
    pingpong::tile<CD, P2, false, SM>(a, a_s, b, b_s, c, M, N, K, tiles_m, tiles_n, tn_first, kb_per_split, ldc, blockIdx.x);
}

template <int CD, bool G, int TM, int S, bool P2 = false>
__global__ __launch_bounds__(THREADS, 1) void fp8_gemm_prefill_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c,
        int M, int N, int K, int tiles_m, int tiles_n, int tn_first, int kb_per_split, int ldc, GroupTable g) {
    prefill_tile<CD, G, TM, S, S, P2>(a, a_s, b, b_s, c, M, N, K, tiles_m, tiles_n, tn_first, kb_per_split, ldc, g, blockIdx.x);
}

// Grouped GEMM over a tile table with slots of up to 256 rows.  A slot with more than 192 rows runs the 256-row
// two-phase kernel (the weights pass through LDS once for up to 256 rows), one with 129 .. 192 rows a 192-row
// configuration whose smaller activation stages leave room for a third weight stage (a group's weights come
// straight from HBM, and a second block of prefetch is what hides that), one with fewer the 128-row
// configuration with three stages of both.  The choice is uniform over the workgroup and needs no host knowledge of
// the group sizes: a layer with a few rows per expert and one with hundreds go through the same launch.
// SCB: the rows of a_s and b_s are whole numbers of aligned 16-byte pieces (K a multiple of 512), so that the tiles
// copy their scales four K blocks at a time.
template <int CD, bool P2 = false, bool SG = false, bool SCB = false>
__global__ __launch_bounds__(THREADS, 1) void fp8_gemm_grouped_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c,
        int M, int N, int K, int tiles_m, int tiles_n, int tn_first, int kb_per_split, int ldc, GroupTable g) {
    const int idx = blockIdx.x / 8, tm = (idx / tiles_n) * 8 + blockIdx.x % 8;
    if (tm >= tiles_m) return;
    const int rows = g.tile_rows[tm];
    if (rows > 192) {
        if (g.tile_group[tm] < 0) return;
        pingpong::tile<CD, P2, true, 4, false, SG, SCB>(a, a_s, b, b_s, c, M, N, K, tiles_m, tiles_n, tn_first, kb_per_split, ldc, blockIdx.x, g);
    }
    else if (rows > 128)
        prefill_tile<CD, true, 192, 2, 3, P2, SG, SCB>(a, a_s, b, b_s, c, M, N, K, tiles_m, tiles_n, tn_first, kb_per_split, ldc, g, blockIdx.x);
    else
        prefill_tile<CD, true, 128, 3, 3, P2, SG, SCB>(a, a_s, b, b_s, c, M, N, K, tiles_m, tiles_n, tn_first, kb_per_split, ldc, g, blockIdx.x);
}

// Dense GEMM whose last column tiles run as 128-row tiles: the first tiles_m * tn_tall workgroups compute 256-row
// tiles over the column tiles [0, tn_tall), the others 128-row tiles over [tn_tall, tn_tall + tn_short).  Workgroups
// are handed out in index order, so the short tiles fill the compute units that the last, partly filled round of
// tall tiles would leave idle.
template <int CD, bool P2 = false, bool PP = true, bool PPS = true>
__global__ __launch_bounds__(THREADS, 1) void fp8_gemm_two_heights_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c, int M, int N, int K, int tn_tall, int tn_short) {
    const int tm_tall = (M + 255) / 256, n_tall = tm_tall * tn_tall;
    const int short_first = (n_tall + 7) & ~7;        // keeps workgroup index % 8 = XCD for the short tiles too
    const GroupTable none{};
    if ((int)blockIdx.x < n_tall) {
        if constexpr (PP) pingpong::tile<CD, P2>(a, a_s, b, b_s, c, M, N, K, tm_tall, tn_tall, 0, K / 128, N, blockIdx.x);
        else prefill_tile<CD, false, 256, 2, 2, P2>(a, a_s, b, b_s, c, M, N, K, tm_tall, tn_tall, 0, K / 128, N, none, blockIdx.x);
    } else if ((int)blockIdx.x >= short_first) {
        if constexpr (PPS) pingpong::tile<CD, P2, false, 2>(a, a_s, b, b_s, c, M, N, K, (M + 127) / 128, tn_short, tn_tall, K / 128, N,
                                                            blockIdx.x - short_first);
        else prefill_tile<CD, false, 128, 3, 3, P2>(a, a_s, b, b_s, c, M, N, K, (M + 127) / 128, tn_short, tn_tall, K / 128, N, none,
                                                    blockIdx.x - short_first);
    }
}

// Dense GEMM of whole 256-row tiles in which wg_tall (a multiple of 8) persistent workgroups walk the tall tiles
// [0, tn_tall) x M / 256, wg_tall apart, with the copies of a tile's first K blocks requested by the last blocks of
// the tile before it (pingpong::tile in persistent mode); the workgroups behind them compute the column tiles
// [tn_tall, tn_tall + tn_short) as 128-row tiles, as in the kernel above.
template <int CD, bool P2 = false>
__global__ __launch_bounds__(THREADS, 1) void fp8_gemm_persistent_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c, int M, int N, int K, int tn_tall, int tn_short, int wg_tall) {
    const GroupTable none{};
    if ((int)blockIdx.x < wg_tall)
        pingpong::tile<CD, P2, false, 4, true>(a, a_s, b, b_s, c, M, N, K, M / 256, tn_tall, 0, K / 128, N, blockIdx.x, none, wg_tall);
    else
        pingpong::tile<CD, P2, false, 2>(a, a_s, b, b_s, c, M, N, K, M / 128, tn_short, tn_tall, K / 128, N, blockIdx.x - wg_tall);
}

}  // namespace prefill

// Usable when the row offsets fit 32 bits; the caller falls back to the generic tile kernel otherwise.
bool prefill_supported(int64_t m, int64_t n, int64_t k) {
    return k >= 128 && m * k < (1ll << 32) && n * k < (1ll << 32);
}

namespace {
// Launches the column tiles [tn_first, tn_first + tn_count) of every row tile.
template <int CD, bool G, int TM, int S, bool P2 = false>
int launch_kernel(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                  int64_t m, int64_t n, int64_t k, int64_t tm, int64_t tn_first, int64_t tn_count,
                  prefill::GroupTable g, hipStream_t stream, int splits = 1, int64_t ldc = 0) {
    using namespace prefill;
    constexpr int LDS_BYTES = Cfg<TM, S>::LDS_BYTES;
    if ((tm + 8) * tn_count > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (tm * tn_count == 0) return DSV3_OK;
    if constexpr (!G && (TM == 256 || TM == 128)) {
        if (TM == 256 ? use_pingpong() : use_pingpong_short()) {
            constexpr int SM = TM / 64, PP_LDS = pingpong::lds_bytes<SM>();
            auto pp = fp8_gemm_pingpong_kernel<CD, P2, SM>;
            static LdsGrant pp_grant;
            if (!pp_grant.ensure((const void*)pp, PP_LDS)) return DSV3_ERR_LAUNCH;
            const int kbt = (int)(k / 128), per = (kbt + splits - 1) / splits;
            hipLaunchKernelGGL(pp, dim3((unsigned)(tm * tn_count), (unsigned)((kbt + per - 1) / per)), dim3(THREADS),
                               PP_LDS, stream, (const uint8_t*)a, a_s, (const uint8_t*)b, b_s,
                               (typename OutT<CD>::type*)c, (int)m, (int)n, (int)k, (int)tm, (int)tn_count, (int)tn_first,
                               per, (int)(ldc ? ldc : n));
            return launch_status();
        }
    }
    auto kern = fp8_gemm_prefill_kernel<CD, G, TM, S, P2>;
    static LdsGrant grant;
    if (!grant.ensure((const void*)kern, LDS_BYTES)) return DSV3_ERR_LAUNCH;
    const int64_t grid = (G ? (tm + 7) / 8 * 8 : tm) * tn_count;       // grouped: row tiles are dealt over the 8 XCDs
    const int kb = (int)(k / 128), kb_per_split = (kb + splits - 1) / splits;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid, (unsigned)((kb + kb_per_split - 1) / kb_per_split)), dim3(THREADS),
                       LDS_BYTES, stream, (const uint8_t*)a, a_s, (const uint8_t*)b, b_s,
                       (typename OutT<CD>::type*)c, (int)m, (int)n, (int)k, (int)tm, (int)tn_count, (int)tn_first,
                       kb_per_split, (int)(ldc ? ldc : n), g);
    return launch_status();
}
constexpr int kGroupedTileRows = 256;     // slot height of the grouped kernel's tile table
// whether the rows of a_s and of every group's b_s (K / 128 binary32 values each) are whole numbers of aligned 16-byte pieces
inline bool scale_batches_ok(const float* a_s, const float* b_s, int64_t bs_stride, int64_t k) {
    return (k / 128) % 4 == 0 && (((uintptr_t)a_s | (uintptr_t)b_s) & 15) == 0 && bs_stride % 4 == 0;
}
constexpr int64_t kCUs = 256;
inline int env_tile_rows() { static const int v = [] { const char* e = getenv("DSV3_PREFILL_TILE"); return e ? atoi(e) : 0; }(); return v; }
}  // namespace

// Tile height, K slicing and the last partial round.  A K block of a 256-row tile costs about 1.64x one of a
// 128-row tile (measured, K = 7168) and the tiles are dealt over 256 compute units in whole rounds.  Four kinds of
// plan, compared by rounds x K blocks per workgroup x per-block cost:
//   plain   all tiles in one launch;
//   sliced  when the tiles do not fill a round: the K range cut into up to 8 slices of at least 8 blocks that run
//           as separate workgroups and write binary32 partial sums ("slabs"), added in a fixed order by a second
//           kernel;
//   hybrid  the column tiles that fill whole rounds as a plain launch, the remaining columns (less than a round
//           of tiles) as a sliced launch -- instead of a last round that leaves most of the chip idle;
//   two heights  tall tiles for the first column tiles and short tiles for the last ones, in ONE launch: the short
//           tiles start on whichever compute unit is free first and fill the partly filled last round.
// (M = 4096 x N = 18432: two heights, 4 rounds of tall tiles + 1 of short ones instead of 5 of tall; M = 1024:
// hybrid, 256 tall tiles + 32 tall tiles in 8 slices; M = 192 ... 256: sliced, 72 tall tiles in 3 slices; M = 128:
// sliced, 72 short tiles.)
namespace {
struct PrefillPlan {
    int tile_rows;      // 128 or 256
    int tn_plain;       // column tiles of the plain launch (0: none)
    int slabs;          // K slices of the remaining column tiles (1 with tn_plain == all: no sliced launch)
    int tn_short;       // two heights: the last tn_short column tiles run as 128-row tiles in the same launch as the
                        // tn_plain tall ones (tile_rows == 256, slabs == 1); 0 otherwise
};

// sums `slabs` binary32 slabs [m, w] into columns [n0, n0 + w) of c [m, n]; 4 columns per thread when aligned
template <int CD>
__global__ __launch_bounds__(256) void slab_reduce_kernel(
        const float* __restrict__ ws, typename OutT<CD>::type* __restrict__ c, int64_t m, int w, int64_t n, int n0,
        int slabs) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;       // element of the [m, w] slab
    const int64_t mw = m * w;
    if (i >= mw) return;
    const int64_t row = i / w;
    const int col = (int)(i - row * w);
    typename OutT<CD>::type* dst = c + row * n + n0 + col;
    if ((w & 3) == 0 && (n & 3) == 0) {
        // all (up to eight) slabs' partial sums are requested before the first addition: a load-then-add loop pays a
        // round trip to L2 per slab.  Slabs past the last are requested again from the last and left out of the sum.
        v4f v = {0.f, 0.f, 0.f, 0.f};
        for (int s0 = 0; s0 < slabs; s0 += 8) {
            v4f t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = *(const v4f*)(ws + (int64_t)min(s0 + u, slabs - 1) * mw + i);
#pragma unroll
            for (int u = 0; u < 8; ++u) v = s0 + u < slabs ? v + t[u] : v;
        }
        if (CD == DSV3_F32) *(v4f*)dst = v;
        else if (CD == DSV3_BF16) *(v2u*)dst = v2u{ pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]) };
        else *(v2u*)dst = v2u{ pack_f16(v[0], v[1]), pack_f16(v[2], v[3]) };
    } else {
        for (int e = 0; e < 4 && i + e < mw; ++e) {
            const int64_t r = (i + e) / w;
            const int cc = (int)(i + e - r * w);
            float v = 0.f;
            for (int s = 0; s < slabs; ++s) v += ws[(int64_t)s * mw + i + e];
            c[r * n + n0 + cc] = cvt_out<CD>(v);
        }
    }
}

PrefillPlan prefill_plan(int64_t m, int64_t n, int64_t k) {
    const int64_t tn = (n + prefill::BN - 1) / prefill::BN, kb = k / 128;
    const int forced = env_tile_rows();
    static const bool nosplit = getenv("DSV3_PREFILL_NOSPLIT") != nullptr;
    PrefillPlan best{128, (int)tn, 1, 0};
    int64_t best_cost = -1;
    // a round of 128-row tiles against one of 256-row tiles (152): 0.60 on the two-phase kernel, 0.66 on the single-phase one
    const int64_t short_unit = prefill::use_pingpong_short() ? 91 : 100;
    auto slices_for = [&](int64_t tiles) {       // K slices that keep `tiles` within one round
        int64_t s = tiles > 0 ? kCUs / tiles : 1;
        if (s > kb / 8) s = kb / 8;
        if (s > 8) s = 8;
        return (s < 2 || nosplit) ? (int64_t)1 : s;
    };
    // a sliced launch also pays for a second launch and for writing and re-reading its binary32 slabs (8 bytes per
    // element and slab at ~6 TB/s), in hundredths of a short tile's K block (1.14 us)
    auto slab_cost = [&](int64_t slabs, int64_t cols) { return 300 + slabs * m * cols * 12 / 100000; };
    for (int h : {128, 256}) {
        if (forced && forced != h) continue;
        const int64_t unit = h == 128 ? short_unit : (prefill::use_pingpong() ? 152 : 164), tm = (m + h - 1) / h, tiles = tm * tn;
        // plain or sliced over all columns
        {
            const int64_t s = slices_for(tiles), per = (kb + s - 1) / s, slabs = (kb + per - 1) / per;
            int64_t cost = ((tiles * slabs + kCUs - 1) / kCUs) * per * unit;
            if (slabs > 1) cost += slab_cost(slabs, n);
            if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = PrefillPlan{h, slabs > 1 ? 0 : (int)tn, (int)slabs, 0}; }
        }
        // hybrid: whole rounds plain, the remaining column tiles sliced
        const int64_t tn_plain = (tiles / kCUs) * kCUs / tm, tn_rest = tn - tn_plain;
        // (only for launches of up to three rounds: behind more rounds the partial one overlaps the skew of the
        // full ones, and two serialised launches measured slower -- M = 4096 x N = 18432: 534 against 515 us)
        if (tn_plain > 0 && tn_rest > 0 && !nosplit && tiles <= 3 * kCUs) {
            const int64_t s = slices_for(tm * tn_rest), per = (kb + s - 1) / s, slabs = (kb + per - 1) / per;
            if (slabs > 1) {
                const int64_t cols = n - tn_plain * prefill::BN;
                const int64_t cost = ((tm * tn_plain + kCUs - 1) / kCUs) * kb * unit + per * unit + slab_cost(slabs, cols) + 300;
                if (cost < best_cost) { best_cost = cost; best = PrefillPlan{h, (int)tn_plain, (int)slabs, 0}; }
            }
        }
    }
    // two heights: the last c column tiles as short tiles behind the tall ones, in one launch.  Workgroups start in
    // index order on the first free compute unit: the tall tiles leave r units with q + 1 tiles and the others with
    // q; the short tiles then fill up from the least loaded unit.
    if (!forced && !nosplit && m > 128) {
        const int64_t tm_tall = (m + 255) / 256, tm_short = (m + 127) / 128;
        for (int64_t c = 1; c < tn && c <= 32; ++c) {
            const int64_t n_tall = tm_tall * (tn - c), n_short = tm_short * c;
            const int64_t q = n_tall / kCUs, r = n_tall % kCUs;
            // kCUs - r units carry lo = q * tall, r units hi = lo + tall; the short tiles (short_unit each) go to whichever
            // unit is free first, level by level
            const int64_t tall = prefill::use_pingpong() ? 152 : 164;
            const int64_t lo = q * tall, hi = lo + tall;
            int64_t t = lo, t_lo = lo + short_unit, t_hi = hi + short_unit, done = 0;
            while (done < n_short) {
                if (r == 0 || t_lo <= t_hi) { t = t_lo; t_lo += short_unit; done += kCUs - r; }
                else                        { t = t_hi; t_hi += short_unit; done += r; }
            }
            const int64_t span = (r > 0 && hi > t) ? hi : t;
            const int64_t cost = span * kb + 100;                // (a little extra: prefer one height at equal cost)
            if (cost * 100 < best_cost * 97) { best_cost = cost; best = PrefillPlan{256, (int)(tn - c), 1, (int)c}; }
        }
    }
    return best;
}
}  // namespace

size_t prefill_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || n <= 0 || k < 128) return 0;
    const PrefillPlan p = prefill_plan(m, n, k);
    if (p.slabs <= 1) return 0;
    const int64_t cols = n - (int64_t)p.tn_plain * prefill::BN;
    return (size_t)p.slabs * (size_t)m * (size_t)cols * sizeof(float);
}

// The persistent kernel takes a plan of 256-row tiles (and, behind them, 128-row tiles) when every tile is whole,
// the K range is an even number of blocks between 4 and 32, the results are 16 bits wide and the tall tiles are more
// than one round.  What it saves is ~3.5 us per tile after a workgroup's first; what it costs is that tiles are dealt
// to the workgroups in advance instead of to whichever compute unit is free, and a per-block ~1 % from the longer
// code.  M = 4096: 512 -> 32768 (8 tiles of 4 blocks per workgroup) 106 -> 91 us, 1536 -> 24576 148 -> 136 us,
// 2048 -> 7168 59 -> 57.5 us, 4096 -> 7168 102.5 -> 101 us; at 56 blocks per tile (7168 -> 18432) the two are equal
// and at 144 (18432 -> 7168, 448 tiles) the fixed deal loses 8 us of 408, hence the upper limit.
// DSV3_PREFILL_NOPERSIST=1 switches it off (tuning aid).  Returns -1 when the plan is not for it.
template <int CD, bool P2>
int launch_persistent(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                      int64_t m, int64_t n, int64_t k, int64_t tn_tall, int64_t tn_short, hipStream_t stream) {
    using namespace prefill;
    if constexpr (CD == DSV3_F32) return -1;
    else {
        static const bool off = getenv("DSV3_PREFILL_NOPERSIST") != nullptr;
        const int64_t kb = k / 128, n_tall = m / 256 * tn_tall;
        if (off || !use_pingpong_short() || m % 256 || n % 8 || (tn_tall + tn_short) * BN > n || kb < 4 || kb > 32 || kb % 2 || n_tall <= kCUs) return -1;
        constexpr int LDS_BYTES = pingpong::LDS_BYTES + pingpong::PS_STAGING;
        static_assert(LDS_BYTES <= 160 * 1024, "LDS of a compute unit");
        auto kern = fp8_gemm_persistent_kernel<CD, P2>;
        static LdsGrant grant;
        if (!grant.ensure((const void*)kern, LDS_BYTES)) return DSV3_ERR_LAUNCH;
        const int64_t grid = kCUs + m / 128 * tn_short;
        if (grid > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(THREADS), LDS_BYTES, stream, (const uint8_t*)a, a_s,
                           (const uint8_t*)b, b_s, (typename OutT<CD>::type*)c, (int)m, (int)n, (int)k, (int)tn_tall, (int)tn_short, (int)kCUs);
        return launch_status();
    }
}

// ws must hold prefill_workspace_bytes(m, n, k) bytes
template <int CD, bool P2>
int launch_prefill(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                   int64_t m, int64_t n, int64_t k, void* ws, hipStream_t stream) {
    const PrefillPlan p = prefill_plan(m, n, k);
    const int64_t tn = (n + prefill::BN - 1) / prefill::BN;
    const int64_t tm = (m + p.tile_rows - 1) / p.tile_rows;
    const prefill::GroupTable none{};
    if (p.tn_short > 0) {
        using namespace prefill;
        const int rc_ps = launch_persistent<CD, P2>(a, a_s, b, b_s, c, m, n, k, p.tn_plain, p.tn_short, stream);
        if (rc_ps >= 0) return rc_ps;
        constexpr int LDS_OLD = Cfg<256, 2>::LDS_BYTES > Cfg<128, 3>::LDS_BYTES ? Cfg<256, 2>::LDS_BYTES : Cfg<128, 3>::LDS_BYTES;
        constexpr int LDS_BYTES = LDS_OLD > pingpong::LDS_BYTES ? LDS_OLD : pingpong::LDS_BYTES;
        const int pp = use_pingpong() ? (use_pingpong_short() ? 2 : 1) : 0;
        auto kern = pp == 2 ? fp8_gemm_two_heights_kernel<CD, P2, true, true>
                  : pp == 1 ? fp8_gemm_two_heights_kernel<CD, P2, true, false> : fp8_gemm_two_heights_kernel<CD, P2, false, false>;
        static LdsGrant grant[3];
        if (!grant[pp].ensure((const void*)kern, LDS_BYTES)) return DSV3_ERR_LAUNCH;
        const int64_t n_tall = (m + 255) / 256 * p.tn_plain;
        const int64_t grid = (n_tall + 7) / 8 * 8 + (m + 127) / 128 * p.tn_short;
        if (grid > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(THREADS), LDS_BYTES, stream, (const uint8_t*)a, a_s,
                           (const uint8_t*)b, b_s, (typename OutT<CD>::type*)c, (int)m, (int)n, (int)k, p.tn_plain, p.tn_short);
        return launch_status();
    }
    auto run = [&](auto cd, void* out, int64_t tn_first, int64_t tn_count, int splits, int64_t ldc) {
        constexpr int OD = decltype(cd)::value;
        if (p.tile_rows == 128)
            return launch_kernel<OD, false, 128, 3, P2>(a, a_s, b, b_s, out, m, n, k, tm, tn_first, tn_count, none, stream, splits, ldc);
        return launch_kernel<OD, false, 256, 2, P2>(a, a_s, b, b_s, out, m, n, k, tm, tn_first, tn_count, none, stream, splits, ldc);
    };
    if (p.tn_plain > 0) {
        int rc = p.tile_rows == 256 ? launch_persistent<CD, P2>(a, a_s, b, b_s, c, m, n, k, p.tn_plain, 0, stream) : -1;
        if (rc < 0) rc = run(std::integral_constant<int, CD>{}, c, 0, p.tn_plain, 1, 0);
        if (rc != DSV3_OK || p.slabs <= 1) return rc;
    }
    if (!ws) return DSV3_ERR_WORKSPACE;
    const int64_t n0 = (int64_t)p.tn_plain * prefill::BN, cols = n - n0;
    const int rc = run(std::integral_constant<int, DSV3_F32>{}, ws, p.tn_plain, tn - p.tn_plain, p.slabs, cols);
    if (rc != DSV3_OK) return rc;
    const int64_t threads = (m * cols + 3) / 4;
    hipLaunchKernelGGL((slab_reduce_kernel<CD>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                       (const float*)ws, (typename OutT<CD>::type*)c, m, (int)cols, n, (int)n0, p.slabs);
    return launch_status();
}

// Rows per tile slot of the grouped kernel: the caller's tile table is built for this height.
int grouped_tile_rows() { return kGroupedTileRows; }

// a: [a_num_rows, k] fp8 with scales a_s; c: [m, n]; group tables as described at GroupTable.  Byte offsets of a
// and of one group's weights must fit 32 bits.
bool grouped_supported(int64_t a_num_rows, int64_t n, int64_t k) {
    return k >= 128 && k % 128 == 0 && n >= 1 && a_num_rows * k < (1ll << 32) && n * k < (1ll << 32);
}

template <int CD, bool P2>
int launch_grouped(const void* a, const float* a_s, const int* a_rows, const void* b, const float* b_s, void* c,
                   int64_t m, int64_t n, int64_t k, int64_t num_tiles, const int* tile_group, const int* tile_row0,
                   const int* tile_rows, int64_t b_stride, int64_t bs_stride, hipStream_t stream) {
    using namespace prefill;
    // few rows in all (an MoE layer at up to ~35 tokens): the weight-streaming kernel fills the chip where
    // groups x 16 tiles would not, and a group of a few rows costs it no 128-row tile (measured on the 256-expert
    // layer: 116 against 157 us at one token, 695 against 766 us at 32, equal at 48-64, slower beyond)
    static const int skinny_max = getenv("DSV3_GROUPED_SKINNY_MAX") ? atoi(getenv("DSV3_GROUPED_SKINNY_MAX")) : 320;
    if (m <= skinny_max)
        return launch_grouped_skinny(a, a_s, a_rows, b, b_s, c, CD, n, k, num_tiles, tile_group, tile_row0, tile_rows,
                                     b_stride, bs_stride, m < num_tiles ? m : num_tiles, stream);
    GroupTable g{tile_group, tile_row0, tile_rows, a_rows, b_stride, bs_stride, nullptr, nullptr, 0};
    constexpr int LDS_BYTES = Cfg<192, 2, 3>::LDS_BYTES_SCB;           // the largest of the three configurations
    static_assert(LDS_BYTES >= pingpong::LDS_BYTES_SCB && LDS_BYTES >= Cfg<128, 3>::LDS_BYTES_SCB &&
                  LDS_BYTES >= Cfg<192, 2, 3>::LDS_BYTES && LDS_BYTES >= Cfg<128, 3>::LDS_BYTES, "LDS of the grouped kernel");
    const int64_t tn = (n + BN - 1) / BN;
    if ((num_tiles + 8) * tn > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (num_tiles * tn == 0) return DSV3_OK;
    const int64_t grid = (num_tiles + 7) / 8 * 8 * tn;                  // row tiles are dealt over the 8 XCDs
    auto launch = [&](auto kern, LdsGrant& grant) {
        if (!grant.ensure((const void*)kern, LDS_BYTES)) return (int)DSV3_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(THREADS), LDS_BYTES, stream, (const uint8_t*)a, a_s,
                           (const uint8_t*)b, b_s, (typename OutT<CD>::type*)c, (int)m, (int)n, (int)k, (int)num_tiles,
                           (int)tn, 0, (int)(k / 128), (int)n, g);
        return launch_status();
    };
    static LdsGrant grant, grant_scb;
    if (scale_batches_ok(a_s, b_s, bs_stride, k)) return launch(fp8_gemm_grouped_kernel<CD, P2, false, true>, grant_scb);
    return launch(fp8_gemm_grouped_kernel<CD, P2>, grant);
}

// The first GEMM of a SwiGLU block with the activation and the re-quantisation in its epilogue (SwiGLU mode above): b
// holds w1 over w3 per group ([2 * inter, k]), y / s receive act_quant(silu(a w1^T) * (a w3^T)).  Only the tile kernels
// have this mode: launches of few rows (the weight-streaming kernel's) are refused and take the two separate calls.
bool grouped_swiglu_supported(int64_t m, int64_t a_num_rows, int64_t inter, int64_t k) {
    static const int skinny_max = getenv("DSV3_GROUPED_SKINNY_MAX") ? atoi(getenv("DSV3_GROUPED_SKINNY_MAX")) : 320;
    return m > skinny_max && inter >= 128 && inter % 128 == 0 && grouped_supported(a_num_rows, 2 * inter, k) &&
           m * inter < (1ll << 32);
}

int launch_grouped_swiglu(const void* a, const float* a_s, const int* a_rows, const void* b, const float* b_s,
                          void* y, float* s, int64_t m, int64_t inter, int64_t k, int64_t num_tiles,
                          const int* tile_group, const int* tile_row0, const int* tile_rows, int64_t b_stride,
                          int64_t bs_stride, int scale_fmt, hipStream_t stream) {
    using namespace prefill;
    GroupTable g{tile_group, tile_row0, tile_rows, a_rows, b_stride, bs_stride, (uint8_t*)y, s,
                 scale_fmt == DSV3_SCALE_FMT_UE8M0 ? 1 : 0};
    constexpr int LDS_BYTES = Cfg<192, 2, 3>::LDS_BYTES_SCB;
    const int64_t tn = inter / 128;
    if ((num_tiles + 8) * tn > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (num_tiles * tn == 0) return DSV3_OK;
    const int64_t grid = (num_tiles + 7) / 8 * 8 * tn;
    auto launch = [&](auto kern, LdsGrant& grant) {
        if (!grant.ensure((const void*)kern, LDS_BYTES)) return (int)DSV3_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(THREADS), LDS_BYTES, stream, (const uint8_t*)a, a_s,
                           (const uint8_t*)b, b_s, (uint16_t*)nullptr, (int)m, (int)(2 * inter), (int)k, (int)num_tiles,
                           (int)tn, 0, (int)(k / 128), (int)(2 * inter), g);
        return launch_status();
    };
    static LdsGrant grant, grant_scb;
    if (scale_batches_ok(a_s, b_s, bs_stride, k)) return launch(fp8_gemm_grouped_kernel<DSV3_BF16, false, true, true>, grant_scb);
    return launch(fp8_gemm_grouped_kernel<DSV3_BF16, false, true>, grant);
}

#define DSV3_INST(CD) \
    template int launch_prefill<CD, false>(const void*, const float*, const void*, const float*, void*, int64_t, int64_t, int64_t, void*, hipStream_t); \
    template int launch_prefill<CD, true>(const void*, const float*, const void*, const float*, void*, int64_t, int64_t, int64_t, void*, hipStream_t); \
    template int launch_grouped<CD, false>(const void*, const float*, const int*, const void*, const float*, void*, int64_t, int64_t, int64_t, \
                                    int64_t, const int*, const int*, const int*, int64_t, int64_t, hipStream_t);                     \
    template int launch_grouped<CD, true>(const void*, const float*, const int*, const void*, const float*, void*, int64_t, int64_t, int64_t, \
                                    int64_t, const int*, const int*, const int*, int64_t, int64_t, hipStream_t);
DSV3_INST(DSV3_BF16)
DSV3_INST(DSV3_F16)
DSV3_INST(DSV3_F32)
#undef DSV3_INST

}  // namespace dsv3
