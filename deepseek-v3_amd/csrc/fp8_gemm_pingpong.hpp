// fp8_gemm, 256 x 256 tile with the two wavefronts of every SIMD in opposite phases (included by
// fp8_gemm_prefill.hip; reference arithmetic: inference/kernel.py:157-166).
//
// Eight wavefronts, 4 along m x 2 along n, each owning 64 (m) x 128 (n) of the tile as 4 x 8 MFMA tiles of 16 x 16
// (one v_mfma 16x16x128 = one 128-wide scale block of K, folded into binary32 accumulators by one FMA per element
// with a_s[m, kb] * b_s[n / 128, kb]).  Wavefront w runs on SIMD w % 4, so the two wavefronts of a SIMD are the two
// column halves ("groups") of one row quarter.  A K block is four phases per wavefront:
//     M1  read the block's activation fragments (64 rows) and the weight fragments of its first 64 columns from LDS
//         into registers, read the block's scales, request global -> LDS copies
//     C1  16 MFMAs on those registers, each followed by the four FMAs of the MFMA issued two earlier
//     M2  read the weight fragments of the other 64 columns, request copies
//     C2  16 MFMAs
// and two workgroup barriers: group 0 passes one after each C phase, group 1 after each M phase.  Between two
// barriers group 0 therefore runs an M phase and then a C phase while group 1 runs a C phase (of the half block
// before) and then an M phase: whenever a wavefront does its LDS and global memory work, the other wavefront of its
// SIMD is in a C phase, and the matrix pipe always has a wavefront to take instructions from.  Group 1's C phases
// run at raised priority (s_setprio): where the two C phases of a SIMD overlap, the arbiter otherwise serves group
// 0's first, group 1's ends late, and its M phase is left with nothing beside it.  The two barriers are the ones
// the data needs (every region of a stage is refilled only after all eight wavefronts have read it, and read only
// after every wavefront has seen its copies land); a barrier after every phase, which also kept the two wavefronts of
// a SIMD strictly apart, cost 11 % more cycles per block (and, the chip being power limited under this kernel,
// 0.5 % more time).
//
// LDS: two stages of [256 rows of A | 256 rows of B] x 128 bytes (the chunk permutation of fp8_gemm_prefill.hip)
// and two slots of scales; block kb lives in stage kb % 2.  Which wavefront copies what, and when, is laid out at
// the copy plan below: per block a wavefront requests four copies of block kb + 1 in M1 and four of block kb + 2 plus
// the scales in M2 (the same number in each of a block's four M phases), every region is refilled only after its
// last reader's phase has ended, and every copy has at least one whole K block of time to land.  Copies retire in
// program order, so "the copies the next readers need have landed" is a vmcnt(n) with n = the number of younger
// copies: 9 at the end of both M phases for group 1, 5 at the end of C2 for group 0.
//
// Grouped mode (G): the tile is a slot of the grouped GEMM's tile table (a row range of one group, multiplied by that
// group's weights, activation rows gathered through a row map) -- used for slots of more than 192 rows.
#pragma once

namespace pingpong {

// One global -> LDS copy of 16 (or 4) bytes per lane: uniform 64-bit base in scalar registers, 32-bit lane offset,
// uniform LDS address through M0 (lane l lands at lds_addr + 16 l).  Written out because the compiler otherwise
// forms a 64-bit address per lane with vector ALU instructions in front of every copy.
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) { return (uint32_t)(uintptr_t)(lptr_t)p; }
__device__ __forceinline__ void copy16(const void* base, uint32_t lane_off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(base), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ void copy4(const void* base, uint32_t lane_off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 :: "v"(lane_off), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// SM: 16-row sub-tiles per wavefront.  4: the 256-row tile described above.  2: a 128-row tile (32 x 128 per
// wavefront, eight MFMAs per C phase) for problems whose row count or tile count does not fill rounds of 256-row
// tiles; its A stage is half as large and all of it is copied by group 1.
template <int SM> struct Geo {
    static_assert(SM == 2 || SM == 4, "128- or 256-row tiles");
    static constexpr int WM = 16 * SM, TM = 4 * WM;
    static constexpr int A_STAGE = TM * 128, B_STAGE = 256 * 128;       // bytes of A / of B per K block
    static constexpr int LDS_A = 0, LDS_B = 2 * A_STAGE, LDS_SC = 2 * A_STAGE + 2 * B_STAGE;
    // copies per wavefront and K block: NM1_G0 / NM1_G1 in M1 (group 0 / 1), NM2 in M2 (plus the scales)
    static constexpr int NM1_G0 = SM == 4 ? 4 : 2, NM1_G1 = 4, NM2 = SM == 4 ? 4 : 3;
    // copies younger than the ones a phase end has to wait for: group 1 after both of its M phases, group 0 after C2
    static constexpr int WAIT_G1 = NM1_G1 + NM2 + 1, WAIT_G0 = NM2 + 1;
};
constexpr int SC_SLOT = 2048, SC_SLOTS = 2;
template <int SM> constexpr int lds_bytes() { return Geo<SM>::LDS_SC + SC_SLOTS * SC_SLOT; }
constexpr int LDS_BYTES = lds_bytes<4>();               // 136 KiB (100 KiB for the 128-row tile)
constexpr int LDS_BYTES_SCB = LDS_BYTES + 3 * 4096;     // with scale batches: two buffers and the area of the copies nobody reads

// PS (persistent): the workgroup computes tiles wg, wg + wg_stride, ... one after the other and treats their K blocks
// as one stream -- the last two blocks of a tile request the first copies of the next tile where a single tile
// repeats its last block, so the next tile starts without a prologue, and the finished tile's results leave through a
// staging area of their own (2 KiB per wavefront behind the scales) while those copies are in flight.  Between two
// tiles of a 7168-deep product this hides ~3 us of first-copy latency, ~0.7 us of workgroup dispatch and most of the
// ~2.5 us a workgroup spends writing its results with nothing else resident on its compute unit.  For whole tiles
// only (M a multiple of 256, the column tiles inside N), an even number (>= 4) of K blocks, one K slice and 16-bit
// results; the caller sends everything else down the one-tile path.
constexpr int PS_STAGING = 8 * 2048;

// SCB (grouped mode): the activation scales are copied four K blocks at a time, see issue_scales.
template <int CD, bool P2, bool G = false, int SM = 4, bool PS = false, bool SG = false, bool SCB = false>
__device__ __forceinline__ void tile(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c,
        int M, int N, int K, int tiles_m, int tiles_n, int tn_first, int kb_per_split, int ldc, int wg,
        const GroupTable& g = GroupTable{}, int wg_stride = 0) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    using GEO = Geo<SM>;
    constexpr int TM = GEO::TM, WM = GEO::WM, A_STAGE = GEO::A_STAGE, B_STAGE = GEO::B_STAGE;
    constexpr int LDS_A = GEO::LDS_A, LDS_B = GEO::LDS_B, LDS_SC = GEO::LDS_SC, NM2 = GEO::NM2;
    static_assert(!G || SM == 4, "grouped slots run the 256-row tile");
    static_assert(!PS || (!G && SM == 4 && CD != DSV3_F32), "persistent mode: dense 256-row tiles with 16-bit results");
    static_assert(!SG || (G && !P2 && CD == DSV3_BF16), "SwiGLU mode: grouped, binary32 scales, bf16 intermediate");

    // ---- workgroup -> tile: a contiguous run of tiles per XCD, walked in bands of GROUP_M tile rows; in grouped
    // mode the row tiles are dealt round-robin over the XCDs and the column tiles of a row tile stay on one XCD
    // (the mapping of the grouped kernel, whose dispatch has already checked that the slot is in use)
    const int T = tiles_m * tiles_n;
    auto dense_origin = [&](int w, int& m0_, int& n0_) {
        int pid = w;
        {
            const int q = T / 8, r = T % 8, x = pid % 8;
            pid = x * q + (x < r ? x : r) + pid / 8;
        }
        constexpr int GROUP_M = 4;
        const int band = pid / (GROUP_M * tiles_n);
        const int band_rows = min(GROUP_M, tiles_m - band * GROUP_M);
        const int in_band = pid - band * GROUP_M * tiles_n;
        m0_ = (band * GROUP_M + in_band % band_rows) * TM;
        n0_ = (tn_first + in_band / band_rows) * BN;
    };
    int m0, n0, rows_here;
    int tn_idx = 0;                     // (SwiGLU mode: the column tile)
    if (G) {
        const int x = wg % 8, idx = wg / 8;
        const int tm = (idx / tiles_n) * 8 + x, tn = idx - (idx / tiles_n) * tiles_n;
        const int expert = g.tile_group[tm];
        m0 = g.tile_row0[tm];
        rows_here = g.tile_rows[tm];
        n0 = (tn_first + tn) * BN;
        tn_idx = tn_first + tn;
        b += (size_t)expert * g.b_stride;
        b_s += (size_t)expert * g.bs_stride;
    } else {
        dense_origin(wg, m0, n0);
        rows_here = min(TM, M - m0);
    }
    // row of a behind row r of the tile; rows past the tile's end repeat its last row (their results are dropped).
    // In persistent mode the tile's origin is part of the copies' scalar base address instead (cur / nxt below).
    const int m0_ld = PS ? 0 : m0, n0_ld = PS ? 0 : n0;
    auto a_row = [&](int r) -> uint32_t {
        const int rr = m0_ld + min(r, rows_here - 1);
        return (uint32_t)((G && g.a_rows) ? g.a_rows[rr] : rr);
    };

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 3, grp = wave >> 2;
    const int KBT = K / 128;
    const int kb0 = blockIdx.y * kb_per_split;
    const int KB = min(kb_per_split, KBT - kb0);
    c += (size_t)blockIdx.y * (size_t)M * (size_t)ldc;
    const int n_base = ldc == N ? 0 : tn_first * BN;
    a += (size_t)kb0 * 128u; b += (size_t)kb0 * 128u;
    // persistent mode: the tile being computed and the one after it (the same once more behind the last one: its
    // copies land in stages nobody reads any more)
    struct Origin { const uint8_t* a; const uint8_t* b; const float* sc; };
    auto origin_of = [&](int m0_, int n0_) {
        return Origin{ a + (size_t)m0_ * (size_t)K, b + (size_t)n0_ * (size_t)K,
                       wave < 4 ? a_s + (size_t)m0_ * (size_t)(K / 128) : b_s + (size_t)(n0_ / 128) * (size_t)(K / 128) };
    };
    int cur_w = wg, m0n = m0, n0n = n0;
    bool has_next = PS && cur_w + wg_stride < T;
    if (has_next) dense_origin(cur_w + wg_stride, m0n, n0n);
    Origin cur = origin_of(m0, n0), nxt = origin_of(m0n, n0n);

    // ---- copy plan.  A K block is TM / 8 + 32 wavefront-copies of 8 rows (1 KiB); copy q covers rows 8q .. 8q + 7.
    // The copies are requested in the M phases, interleaved with the LDS reads (the copy path takes one 1 KiB copy
    // per ~16 cycles and compute unit and holds the issuing wavefront meanwhile; a wavefront in a C phase that
    // issued them would leave gaps in its MFMA stream), and spread evenly over the four M phases of a K block (two
    // per group): with most of them in the M2 phases the second of the two found the memory pipeline still full of
    // the first one's requests and took 140 cycles longer than the C phase beside it.
    // What may be requested when: the part of a stage that M1 reads (all of A, B rows 0-63 and 128-191, the scales)
    // is free once group 1 has left M1 of block kb and is read again by group 0 in M1 of block kb + 2 -- it is
    // refilled in M2 of block kb by both groups and in M1 of block kb + 1 by group 0; the part that M2 reads (B
    // rows 64-127 and 192-255) is free once group 1 has left M2 of block kb, and group 1 refills it in M1 of
    // block kb + 1.  Per block kb a wavefront therefore issues
    //   in M1  copies of block kb + 1:  group 1  B rows 64-127 and 192-255 (4 per wavefront)
    //                                   group 0  the last 4 NM1_G0 entries of the list below
    //   in M2  copies of block kb + 2:  group 0  entries 0 .. 4 NM2 - 1, group 1  entries 4 NM2 .. 8 NM2 - 1 of the list
    //          [B rows 0-63, B rows 128-191, A rows 0 .. TM - 1] in groups of 8 rows, and the scales
    // (256-row tile: 4 + 4 per wavefront and block, group 0 copies B's first halves and A rows 128-255, group 1 A rows
    // 0-127; 128-row tile: 2 + 3 and 4 + 3).
    constexpr int NM1_G0 = GEO::NM1_G0, NM1_G1 = GEO::NM1_G1, NM1 = NM1_G0 > NM1_G1 ? NM1_G0 : NM1_G1;
    static_assert(8 * NM2 + 4 * NM1_G0 == 16 + TM / 8 && 4 * NM1_G1 == 16, "every 8-row group of a K block is copied once");
    // per copy: the lane's source offset, the LDS address in stage 0 and in stage 1 (the two regions' stages differ in
    // size in the 128-row tile), and whether it comes from b
    uint32_t m1_src[NM1], m2_src[NM2];
    uint32_t m1_dst[2][NM1], m2_dst[2][NM2];
    bool m1_from_b[NM1], m2_from_b[NM2];
    const uint32_t lds0 = lds_addr_of(lds);
    auto plan = [&](bool from_b, int q, uint32_t& src, uint32_t& dst0, uint32_t& dst1) {
        const int r = q * 8 + (lane >> 3), ch = (lane & 7) ^ swz(r);
        src = (from_b ? (uint32_t)(SG ? sg_weight_row(r, tn_idx, N / 2) : min(n0_ld + r, N - 1)) : a_row(r)) * (uint32_t)K + ch * 16;
        dst0 = lds0 + (from_b ? LDS_B : LDS_A) + q * 1024;
        dst1 = dst0 + (from_b ? B_STAGE : A_STAGE);
    };
    // entry idx of the list [B rows 0-63, B rows 128-191, A rows 0 .. TM - 1]
    auto plan_listed = [&](int idx, uint32_t& src, uint32_t& dst0, uint32_t& dst1, bool& from_b) {
        from_b = idx < 16;
        plan(from_b, from_b ? (idx < 8 ? idx : idx + 8) : idx - 16, src, dst0, dst1);
    };
#pragma unroll
    for (int t = 0; t < NM1; ++t) {
        const int listed = 8 * NM2 + wm * NM1_G0 + min(t, NM1_G0 - 1);
        const bool fb = grp == 1 || listed < 16;
        const int q = grp == 1 ? (t < 2 ? 8 : 24) + wm * 2 + (t & 1) : (listed < 16 ? (listed < 8 ? listed : listed + 8) : listed - 16);
        m1_from_b[t] = fb;
        plan(fb, q, m1_src[t], m1_dst[0][t], m1_dst[1][t]);
    }
#pragma unroll
    for (int t = 0; t < NM2; ++t) plan_listed((grp * 4 + wm) * NM2 + t, m2_src[t], m2_dst[0][t], m2_dst[1][t], m2_from_b[t]);
    // (persistent mode: block KB + i is block i of the next tile; only a tile's last two blocks -- `tail` -- get there)
    auto issue_m1 = [&](int t, int kb, int stage, bool tail = true) {
        if constexpr (PS) {
            const bool nx = tail && kb >= KB;
            copy16((m1_from_b[t] ? (nx ? nxt.b : cur.b) : (nx ? nxt.a : cur.a)) + (uint32_t)(nx ? kb - KB : kb) * 128u, m1_src[t], m1_dst[stage][t]);
        } else copy16((m1_from_b[t] ? b : a) + (uint32_t)kb * 128u, m1_src[t], m1_dst[stage][t]);
    };
    auto issue_m2 = [&](int t, int kb, int stage, bool tail = true) {
        if constexpr (PS) {
            const bool nx = tail && kb >= KB;
            copy16((m2_from_b[t] ? (nx ? nxt.b : cur.b) : (nx ? nxt.a : cur.a)) + (uint32_t)(nx ? kb - KB : kb) * 128u, m2_src[t], m2_dst[stage][t]);
        } else copy16((m2_from_b[t] ? b : a) + (uint32_t)kb * 128u, m2_src[t], m2_dst[stage][t]);
    };
    // scales of a K block: wavefronts 0-3 copy a_s[row, kb] of 64 tile rows each, wavefront 4 the b_s rows of the two
    // column halves (lanes 0 and 1; its other lanes and wavefronts 5-7 repeat an address already requested, so that
    // every wavefront issues the same number of copies per block without asking the memory pipeline for more lines).
    // a_s[row, kb] sits 4 KBT bytes from a_s[row + 1, kb]: the 64 scales of a copy are 64 memory lines, a third of all
    // the lines a workgroup asks for, and they slow the phase after the one that requests them by 80-100 cycles (with
    // one line per copy, results aside, a K block of a dense problem takes 2 % less).  Copying them for four K blocks at
    // a time (16 bytes per row, a one-line copy in the other three blocks to keep the counts) was not faster there, where
    // both operands come from the caches; in grouped mode it is (below).
    const int nb_last = (N - 1) / 128;
    const float* sc_base = wave < 4 ? a_s : b_s;
    const int b_scale_row = SG ? sg_scale_row(wave == 4 ? min(lane, 1) : 0, tn_idx, N / 2)
                               : min((PS ? 0 : n0 / 128) + (wave == 4 ? min(lane, 1) : 0), nb_last);
    const uint32_t sc_off = (wave < 4 ? a_row(wave * 64 + lane) * (uint32_t)KBT : (uint32_t)b_scale_row * (uint32_t)KBT) + (uint32_t)kb0;
    // Grouped mode streams its weights from HBM, and there the 256 lines per K block of the activation scales cost a
    // tenth of a 256-row slot's time (with one line per copy, results aside: 2.24 -> 2.00 us per K block).  When a row
    // of a_s is a whole number of 16-byte pieces, wavefronts 0-3 therefore copy the scales of FOUR K blocks at a time
    // (16 bytes per row, into one of two 4 KiB buffers behind the slots) in the block that would have requested the
    // first of them, and a one-line copy nobody reads in the other three, which keeps the counted waits as they are.
    // (sc_one_line: a 16-byte aligned address of a_s that every lane may read.)
    constexpr int LDS_SCB = LDS_SC + SC_SLOTS * SC_SLOT, SCB_BYTES = 256 * 16;
    constexpr bool batched = SCB;                       // (the caller has checked: KBT % 4 == 0, a_s 16-byte aligned)
    static_assert(!SCB || (G && !PS), "scale batches: grouped mode");
    const uint32_t sc_one_line = (uint32_t)__builtin_amdgcn_readfirstlane((int)sc_off);
    auto issue_scales = [&](int kb, int slot, bool tail = true) {
        if constexpr (batched) if (wave < 4) {
            // (no branch: one in the middle of a phase splits the region the phases' instruction order is pinned in, and
            // the register allocation with it.  The copy that is not needed reads one line and lands in a dump area.)
            const bool real = (kb & 3) == 0;
            const uint32_t off = real ? sc_off * 4u : sc_one_line * 4u;
            const uint32_t dst = lds_addr_of(lds + LDS_SCB) + (real ? ((kb >> 2) & 1) * SCB_BYTES : 2 * SCB_BYTES) + wave * 1024;
            copy16(sc_base + (uint32_t)(real ? kb : 0), off, dst);
            return;
        }
        if constexpr (PS) {
            const bool nx = tail && kb >= KB;
            copy4((nx ? nxt.sc : cur.sc) + (uint32_t)(nx ? kb - KB : kb), sc_off * 4u, lds_addr_of(lds + LDS_SC + slot * SC_SLOT + wave * 256));
        } else copy4(sc_base + (uint32_t)kb, sc_off * 4u, lds_addr_of(lds + LDS_SC + slot * SC_SLOT + wave * 256));
    };

    // ---- fragment addresses: lane reads row (lane & 15) of a 16-row sub-tile, K bytes 32 (lane >> 4) .. + 31
    const int fr = lane & 15, fq = lane >> 4;
    const int fx = swz(fr);
    const int c0 = ((2 * fq) ^ fx) * 16, c1 = ((2 * fq + 1) ^ fx) * 16;
    const uint8_t* a_rd = lds + LDS_A + (wm * WM + fr) * 128;           // + j * 2048 + stage * A_STAGE
    const uint8_t* b_rd = lds + LDS_B + (grp * 128 + fr) * 128;         // + i * 2048 + stage * B_STAGE
    const uint8_t* sa_rd = lds + LDS_SC + (wm * WM + fr) * 4;           // + j * 64 + slot * SC_SLOT
    const uint8_t* sab_rd = lds + LDS_SCB + (wm * WM + fr) * 16;        // (batched) + j * 256 + buffer + 4 (kb & 3)
    const uint8_t* sb_rd = lds + LDS_SC + (256 + grp) * 4;

    v4f acc[8][SM];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < SM; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    // persistent mode: results of the current tile, one 16-row sub-tile and 64 columns at a time: four 16 x 16
    // accumulator tiles go to the wavefront's staging area as 16 rows of 128 bytes (16-byte chunks permuted by the row so
    // that neither the 8-byte writes nor the 16-byte reads collide) and leave as two stores of 8 rows x 128 bytes;
    // the accumulators are cleared for the next tile on the way
    auto ps_epilogue = [&]() {
        uint8_t* stg = lds + LDS_SC + SC_SLOTS * SC_SLOT + wave * 2048;
        const int rr = lane >> 3, ch = lane & 7;
#pragma unroll
        for (int j = 0; j < SM; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    v4f& v = acc[h * 4 + ii][j];
                    v2u o;
                    if (CD == DSV3_BF16) o = v2u{ pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]) };
                    else o = v2u{ pack_f16(v[0], v[1]), pack_f16(v[2], v[3]) };
                    *(v2u*)(stg + fr * 128 + (((ii * 2 + (fq >> 1)) ^ (fr & 7)) * 16) + (fq & 1) * 8) = o;
                    v = (v4f){0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    const int lr = p * 8 + rr;
                    const v4u v = *(const v4u*)(stg + lr * 128 + ((ch ^ (lr & 7)) * 16));
                    *(v4u*)(c + (size_t)(m0 + wm * WM + j * 16 + lr) * N + n0 + grp * 128 + h * 64 + ch * 8) = v;
                }
            }
    };

#define DSV3_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
    auto run = [&](auto gtag) {
        constexpr int GRP = decltype(gtag)::value;
        // prologue: blocks 0 and 1 as far as the steady state expects them to have been requested
#pragma unroll
        for (int t = 0; t < NM2; ++t) issue_m2(t, 0, 0);
        issue_scales(0, 0);
#pragma unroll
        for (int t = 0; t < (GRP == 0 ? NM1_G0 : NM1_G1); ++t) issue_m1(t, 0, 0);
#pragma unroll
        for (int t = 0; t < NM2; ++t) issue_m2(t, min(1, KB - 1), 1);
        issue_scales(min(1, KB - 1), 1);
        __builtin_amdgcn_s_waitcnt(0x0f70);                         // vmcnt(0)
        wg_barrier();

        v8i af[SM], bf[4];
        v4f p14 = {0.f, 0.f, 0.f, 0.f}, p15 = {0.f, 0.f, 0.f, 0.f}; // raw products of the last two MFMAs of a C phase
        float sc[2][SM];                                            // fold factors of even / odd blocks
        int ea[SM], eb = 0;                                         // P2: biased exponents of the block's scales
#pragma unroll
        for (int j = 0; j < SM; ++j) { sc[0][j] = sc[1][j] = 0.f; ea[j] = 0; }

        // 4 SM MFMAs over column sub-tiles I0 .. I0 + 3 with the fold factors s; every MFMA is followed by the four
        // FMAs of the MFMA issued two earlier -- the first two by those of the previous C phase's last two MFMAs
        // (column sub-tile IT, fold factors st), so that the M phases hold no vector ALU work: while the other
        // wavefront of the SIMD is in a C phase, the vector ALU issues this wavefront's instructions only in the gaps.
        auto compute = [&](auto i0_tag, auto it_tag, const float (&s)[SM], const float (&st)[SM]) {
            constexpr int I0 = decltype(i0_tag)::value, IT = decltype(it_tag)::value;
            constexpr int NT = 4 * SM;
            // activation sub-tile of MFMA t: the SM sub-tiles are walked forwards for even weight fragments and
            // backwards for odd ones, so that consecutive instructions always share one operand (measured 0.5 %)
            auto SJ = [](int t) { return ((t / SM) & 1) ? SM - 1 - (t % SM) : (t % SM); };
            __builtin_amdgcn_sched_barrier(0);
            if (GRP == 1) __builtin_amdgcn_s_setprio(3);
            if constexpr (P2) {
#pragma unroll
                for (int ii = 0; ii < 4; ++ii)
#pragma unroll
                    for (int j = 0; j < SM; ++j)
                        acc[I0 + ii][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            bf[ii], af[j], acc[I0 + ii][j], 0, 0, 0, eb, 0, ea[j]);
            } else {
                const v4f z = {0.f, 0.f, 0.f, 0.f};
                v4f p[NT];
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    p[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[t / SM], af[SJ(t)], z, 0, 0, 0, 0, 0, 0);
                    if (t < 2) {
                        const v4f q = t == 0 ? p14 : p15;
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[IT][SJ(NT - 2 + t)][e] = __builtin_fmaf(q[e], st[SJ(NT - 2 + t)], acc[IT][SJ(NT - 2 + t)][e]);
                    } else {
                        const int u = t - 2;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc[I0 + u / SM][SJ(u)][e] = __builtin_fmaf(p[u][e], s[SJ(u)], acc[I0 + u / SM][SJ(u)][e]);
                    }
                    DSV3_SGB(0x008, 1);
                    DSV3_SGB(0x002, 4);
                }
                p14 = p[NT - 2]; p15 = p[NT - 1];
            }
            if (GRP == 1) __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
        };

        // one K block whose LDS stage (and scale slot) ST is a compile-time constant: every LDS address of the loop is
        // a register plus an immediate
        auto block = [&](int kb, auto st_tag, auto tail_tag) {
            constexpr int ST = decltype(st_tag)::value;
            constexpr bool TAIL = decltype(tail_tag)::value;     // persistent mode: one of the tile's last two blocks
            // (the block numbers behind the copies' addresses are made opaque at the start of the phase that uses
            // them: the scalar arithmetic that follows from them is otherwise moved up, in front of the barrier
            // that ends the C phase before, where the matrix pipe waits for it)
            int kb_m1 = kb;
            asm volatile("" : "+s"(kb_m1));
            const int kb1 = PS ? kb_m1 + 1 : min(kb_m1 + 1, KB - 1);
            // ---- M1
            {
                const uint8_t* as_base = a_rd + ST * A_STAGE;
                const uint8_t* bs_base = b_rd + ST * B_STAGE;
                // copy t goes in front of fragment read t (SM + 4) / n of the phase's SM + 4
                constexpr int N1 = GRP == 0 ? NM1_G0 : NM1_G1;
#pragma unroll
                for (int j = 0; j < SM; ++j) {
#pragma unroll
                    for (int t = 0; t < N1; ++t)
                        if (t * (SM + 4) / N1 == j) issue_m1(t, kb1, ST ^ 1, TAIL);
                    af[j] = join(*(const v4i*)(as_base + j * 2048 + c0), *(const v4i*)(as_base + j * 2048 + c1));
                }
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
#pragma unroll
                    for (int t = 0; t < N1; ++t)
                        if (t * (SM + 4) / N1 == SM + ii) issue_m1(t, kb1, ST ^ 1, TAIL);
                    bf[ii] = join(*(const v4i*)(bs_base + ii * 2048 + c0), *(const v4i*)(bs_base + ii * 2048 + c1));
                }
            }
            {
                const float bs = *(const float*)(sb_rd + ST * SC_SLOT);
                const uint8_t* sab_kb = sab_rd + (((kb >> 2) & 1) * SCB_BYTES + (kb & 3) * 4);
#pragma unroll
                for (int j = 0; j < SM; ++j) {
                    float as;
                    if constexpr (batched) as = *(const float*)(sab_kb + j * 256);
                    else as = *(const float*)(sa_rd + j * 64 + ST * SC_SLOT);
                    if (P2) ea[j] = (int)(f32_as_u32(as) >> 23);
                    else sc[ST][j] = as * bs;
                }
                if (P2) eb = (int)(f32_as_u32(bs) >> 23);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (GRP == 1) __builtin_amdgcn_s_waitcnt(0x0f70 | GEO::WAIT_G1);
            if (GRP == 1) wg_barrier();
            // ---- C1 (its first two FMA groups belong to C2 of the previous block: zeros at kb = 0)
            compute(std::integral_constant<int, 0>{}, std::integral_constant<int, 7>{}, sc[ST], sc[ST ^ 1]);
            if (GRP == 0) wg_barrier();                   // (nothing group 0 has requested is read in the next phase)
            // ---- M2
            {
                int kb_m2 = kb;
                asm volatile("" : "+s"(kb_m2));
                const int kb2 = PS ? kb_m2 + 2 : min(kb_m2 + 2, KB - 1);
                const uint8_t* bs_base = b_rd + ST * B_STAGE + 4 * 2048;
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    if (ii < NM2) issue_m2(ii, kb2, ST, TAIL);
                    bf[ii] = join(*(const v4i*)(bs_base + ii * 2048 + c0), *(const v4i*)(bs_base + ii * 2048 + c1));
                }
                issue_scales(kb2, ST, TAIL);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (GRP == 1) __builtin_amdgcn_s_waitcnt(0x0f70 | GEO::WAIT_G1);
            if (GRP == 1) wg_barrier();
            // ---- C2
            compute(std::integral_constant<int, 4>{}, std::integral_constant<int, 3>{}, sc[ST], sc[ST]);
            if (GRP == 0) __builtin_amdgcn_s_waitcnt(0x0f70 | GEO::WAIT_G0);
            if (GRP == 0) wg_barrier();
        };

        for (;;) {                                                  // (one pass unless persistent)
            constexpr std::integral_constant<int, 0> st0{};
            constexpr std::integral_constant<int, 1> st1{};
            int kb = 0;
            if constexpr (PS) {                                     // (an even number of blocks, at least four)
                for (; kb + 3 < KB; kb += 2) {
                    block(kb, st0, std::false_type{});
                    block(kb + 1, st1, std::false_type{});
                }
                block(kb, st0, std::true_type{});
                block(kb + 1, st1, std::true_type{});
            } else {
                for (; kb + 1 < KB; kb += 2) {
                    block(kb, st0, std::false_type{});
                    block(kb + 1, st1, std::false_type{});
                }
                if (kb < KB) block(kb, st0, std::false_type{});
            }
            // the FMAs of the last two MFMAs
            if (!P2) {
                const int last = (KB - 1) & 1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[7][1][e] = __builtin_fmaf(p14[e], last ? sc[1][1] : sc[0][1], acc[7][1][e]);
                    acc[7][0][e] = __builtin_fmaf(p15[e], last ? sc[1][0] : sc[0][0], acc[7][0][e]);
                }
            }
            if constexpr (!PS) break;
            else {
                // the tile's results leave through this wavefront's own staging area (no barrier: the other group
                // is one phase behind and meets this wavefront again at the next tile's first barrier); then the
                // next tile, whose first two blocks have been requested by the blocks just finished
                ps_epilogue();
                if (!has_next) break;
                cur_w += wg_stride;
                m0 = m0n; n0 = n0n; cur = nxt;
                has_next = cur_w + wg_stride < T;
                if (has_next) { dense_origin(cur_w + wg_stride, m0n, n0n); nxt = origin_of(m0n, n0n); }
                p14 = p15 = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < SM; ++j) sc[0][j] = sc[1][j] = 0.f;
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);                         // the clamped refills of the last blocks
    };
    if (grp == 0) run(std::integral_constant<int, 0>{});
    else          run(std::integral_constant<int, 1>{});
#undef DSV3_SGB
    if constexpr (PS) return;

    // ---- epilogue: lane holds c[m][n .. n + 3] for every (i, j); see fp8_gemm_prefill.hip for the LDS route
    constexpr int WN = 128, SN = 8;
    auto sub_row = [&](int j) { return wm * WM + j * 16; };
    if constexpr (SG) {
        swiglu_store<SM>(acc, lds, wm, grp, lane, sub_row, m0, rows_here, tn_idx, N / 2, g);
        return;
    }
    const bool lds_epilogue = CD != DSV3_F32 && (N % 8) == 0 && ldc == N;
    const bool f32_lds_epilogue = CD == DSV3_F32 && (N % 4) == 0 && (ldc % 4) == 0;
    const bool vec_ok = (N % 4) == 0 && (ldc % 4) == 0;
    if (lds_epilogue) {
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
            const int lr = p * 4 + rr;
            const v4u v = *(const v4u*)(stg + lr * 256 + ((ch ^ (lr & 15)) * 16));
            const int r = sub_row(lr >> 4) + (lr & 15);
            const int n = n0 + grp * WN + ch * 8;
            if (r < rows_here && n < N)
                *(v4u*)(c + (size_t)(m0 + r) * N + n) = v;
        }
        return;
    }
    if (f32_lds_epilogue) {
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
                const int n = n0 + grp * WN + h * (WN / 2) + ch * 4;
                if (r < rows_here && n < N)
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
            const int n = n0 + grp * WN + i * 16 + fq * 4;
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

}  // namespace pingpong
