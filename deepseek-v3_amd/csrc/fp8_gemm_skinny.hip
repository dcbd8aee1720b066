// fp8_gemm for decode shapes (M <= 64) on gfx950: a weight-streaming kernel
// (reference arithmetic: inference/kernel.py:145-172).
//
//   c[m,n] = sum_kb ( sum_{t<128} a[m,128kb+t] * b[n,128kb+t] ) * a_s[m,kb] * b_s[n/128,kb]
//
// With M <= 64 every weight byte is used once, so the kernel is bound by how
// fast b can be pulled out of HBM.  There is no reuse to stage: each wavefront
// loads its weight rows straight from global memory into the register layout of
// v_mfma_f32_16x16x128_f8f6f4 (lane l holds row l%16, 32 bytes of the K block)
// and keeps several K blocks of loads in flight.  The activations (at most
// 64 x K bytes, shared by every wavefront) come through the vector L1/L2.
//
// Work split: a workgroup owns 16*S weight rows and a contiguous range of K
// blocks (grid.y = split over K across workgroups); inside the workgroup the
// wavefronts split that range again and their partial sums are added in LDS in
// a fixed order, so the result does not depend on timing.  With more than one
// workgroup along K the partial [M,N] slabs go to the caller's workspace and a
// second kernel adds them, again in a fixed order.
//
// Both MFMA operands take their 32 bytes per lane from the same K offsets
// ({16q..16q+15} and {64+16q..64+16q+15}, q = lane/16), chosen so that the four
// lanes that share a row read 64 contiguous bytes per load instruction.
#include <cstdlib>
#include "common.hpp"

namespace dsv3 {
namespace skinny {

constexpr int kMaxWaves = 16;


__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    v8i r = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
    return r;
}

// a = what the lane loaded from rows 0..7, b = from rows 8..15 (see the weight loads in the kernel).  Lanes with
// (lane & 15) < 8 own a row of the first group: their fragment is [a, b-of-lane^8 ... no: a-of-lane^8's second half];
// written out: first 16 bytes  = lane<8 ? a : ror8(b);  last 16 bytes = lane<8 ? ror8(a) : b.
__device__ __forceinline__ v8i untangle(v4i a, v4i b) {
    v8i r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // row_ror:8 inside each 16-lane row; bank_mask picks the lanes that take the rotated value
        r[i]     = __builtin_amdgcn_update_dpp(a[i], b[i], 0x128, 0xf, 0xc, false);
        r[4 + i] = __builtin_amdgcn_update_dpp(b[i], a[i], 0x128, 0xf, 0x3, false);
    }
    return r;
}

// measured on gfx950: 16 consecutive lanes reading one logical 16-byte chunk of 16 consecutive 128-byte LDS rows
// do not collide when the chunk index is xor-ed with this function of the row
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// MT: 16-row activation sub-tiles (M <= 16*MT); S: 16-row weight strips per wavefront;
// NPF: K blocks of weight loads kept in flight per wavefront.
//
// The workgroup first copies the activations of its whole K range (and their scales) into LDS; the wavefronts
// then read them with ds_read while the weight loads stream through a register ring.  LDS reads and vector
// memory loads retire on different counters, so fetching an activation never drains the weight ring.
constexpr int kSlabChunks = 4;             // 16-byte activation chunks a thread stages on the way to LDS

// QF (fused linear, inference/model.py:159-160): `a` holds the bf16 activations themselves and a_s is unused; the
// workgroup quantises its K range of them on the way into LDS exactly as act_quant would (amax over the 128
// block, clamp at 1e-4, / 448, optional power-of-two rounding of the scale, correctly rounded quotient, OCP e4m3),
// so the result equals act_quant followed by this kernel bit for bit and the separate launch disappears.
// 16-byte non-temporal load from (scalar base + 32-bit lane offset + immediate), and a wait until at most n vector
// loads of the wavefront are outstanding with the ring slot threaded through it (so that the slot's consumers cannot
// be scheduled ahead of the wait): the RING variant's weight loads and waits are written out, because the compiler's
// own counting of outstanding loads falls back to "all of them" across a loop's back edge.
#define DSV3_GLOAD(dst, voff, sbase, imm) \
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:" #imm " nt" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory")
#define DSV3_WAIT(n, lo, hi) asm volatile("s_waitcnt vmcnt(" #n ")" : "+v"(lo), "+v"(hi) :: "memory")
template <int N> struct WaitFor;
#define DSV3_WAITFOR(N_) template <> struct WaitFor<N_> { static __device__ __forceinline__ void on(v4i& lo, v4i& hi) { DSV3_WAIT(N_, lo, hi); } };
DSV3_WAITFOR(0) DSV3_WAITFOR(2) DSV3_WAITFOR(4) DSV3_WAITFOR(6) DSV3_WAITFOR(8) DSV3_WAITFOR(10) DSV3_WAITFOR(12) DSV3_WAITFOR(14)
#undef DSV3_WAITFOR

// RING (S == 1, every wavefront's K range a multiple of NPF blocks and at least two of them, n k < 2^32): a ring slot
// is refilled as soon as its block has been multiplied, so a wavefront keeps NPF blocks of loads in flight until its
// last NPF blocks.  Without it the range is worked through in batches -- issue NPF, use NPF, issue the next NPF --,
// a wavefront has nothing in flight while it uses a batch, and all wavefronts of the chip reach that point together.
template <int MT, int S, int NPF, bool QF, bool RING = false>
__global__ __launch_bounds__(kMaxWaves * kWave) __attribute__((amdgpu_waves_per_eu(4, 4))) void fp8_gemm_skinny_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        void* __restrict__ out, int out_dtype,      // out_dtype: dsv3_dtype of `out` (F32 slabs when gridDim.y > 1)
        int M, int N, int K, int kb_per_wg, int ue8m0, uint64_t m_magic) {     // m_magic = ceil(2^32 / M)
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_waves = blockDim.x >> 6;
    const int KB = K >> 7;
    const int fr = lane & 15, fq = lane >> 4;

    // K blocks of this workgroup, then of this wavefront
    const int wg_kb0 = blockIdx.y * kb_per_wg;
    const int wg_nkb = min(kb_per_wg, KB - wg_kb0);
    const int per_wave = (wg_nkb + n_waves - 1) / n_waves;
    const int kb0 = wg_kb0 + wave * per_wave;                 // first K block of the wavefront (global index)
    const int nkb = max(0, min(per_wave, wg_kb0 + wg_nkb - kb0));

    const int n0 = blockIdx.x * (16 * S);
    // Weight loads: an instruction fetches 8 rows x 128 contiguous bytes (lanes with fr < 8 take the first 64
    // bytes of row fr&7, lanes with fr >= 8 the last 64 bytes of the same row); a second one does rows 8..15.
    // The halves that landed in the wrong lane are exchanged between lanes fr and fr^8 with DPP row rotates
    // when the fragment is assembled.  (One instruction per 16 rows x 64 bytes would put the data straight into
    // MFMA layout but reaches markedly less HBM bandwidth.)
    const uint8_t* wsrc[S];
#pragma unroll
    for (int s = 0; s < S; ++s)
        wsrc[s] = b + (size_t)min(n0 + s * 16 + (fr & 7), N - 1) * K + (size_t)kb0 * 128 + (fr >> 3) * 64 + fq * 16;
    // rows 8..15 of the strip: +8 rows, clamped to the last row of b
    size_t wrow8[S];
#pragma unroll
    for (int s = 0; s < S; ++s)
        wrow8[s] = (size_t)(min(n0 + s * 16 + (fr & 7) + 8, N - 1) - min(n0 + s * 16 + (fr & 7), N - 1)) * K;

    // ---- activations of the workgroup's K range -> LDS, packed: slab row kb*M + m holds the 128 bytes of
    // activation row m in K block kb (16-byte chunks permuted by swz(slab row)); the scales follow as
    // [kb*M + m] floats.  A fragment read always spans 16 consecutive slab rows; when M is not a multiple of
    // 16 the surplus rows belong to the next K block (or to the 16 rows of padding at the end) and only feed
    // output columns that are never stored.
    // Their loads are issued first: vector loads retire in issue order, so the slab can be written to LDS while
    // the (younger) weight loads below are still in flight.
    const int slab_rows = kb_per_wg * M + 16;
    uint8_t* act = lds;
    float* act_s = (float*)(lds + (size_t)slab_rows * 128);
    const int chunks = wg_nkb * M * 8;                         // 16-byte chunks to copy (<= kSlabChunks * threads)
    v4i stage[kSlabChunks];
    v4u raw[QF ? kSlabChunks : 1][2];                          // QF: the 16 bf16 values behind each chunk
    float stage_q[QF ? kSlabChunks : 1];                       // QF: weight-block scale of the chunk's K block
    // the two factors of a (row, K block) scale stay apart until the slab is written: multiplying them here would
    // put a wait for these loads in front of the weight loads below
    float stage_sa = 0.f, stage_sb = 0.f;
    // x / M and x % M for x < 2^16 without an integer division (M is a run-time value)
    auto div_m = [&](int x) { return (int)(((uint64_t)(uint32_t)x * m_magic) >> 32); };
#pragma unroll
    for (int i = 0; i < kSlabChunks; ++i) {
        const int c = tid + i * (int)blockDim.x;
        if (c < chunks) {
            const int ch = c & 7, R = c >> 3, kb = div_m(R), row = R - kb * M;
            if (QF) {
                const v4u* src = (const v4u*)(a + 2 * ((size_t)row * K + (size_t)(wg_kb0 + kb) * 128 + ch * 16));
                raw[i][0] = src[0];
                raw[i][1] = src[1];
                stage_q[i] = b_s[(size_t)min(n0 >> 7, (N - 1) >> 7) * KB + wg_kb0 + kb];
            } else {
                stage[i] = *(const v4i*)(a + (size_t)row * K + (size_t)(wg_kb0 + kb) * 128 + ch * 16);
            }
        } else if (QF) {
            raw[i][0] = raw[i][1] = v4u{0u, 0u, 0u, 0u};
            stage_q[i] = 0.f;
        }
    }
    if (!QF && tid < wg_nkb * M) {  // scale of (row, K block) and the weight block's scale
        const int kb = div_m(tid), row = tid - kb * M;
        stage_sa = a_s[(size_t)row * KB + wg_kb0 + kb];
        stage_sb = b_s[(size_t)min(n0 >> 7, (N - 1) >> 7) * KB + wg_kb0 + kb];
    }
    // ---- start the weight stream: the first NPF K blocks of every strip
    v4i wlo[NPF][S], whi[NPF][S];
    auto fetch = [&](int p, int k) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            wlo[p][s] = __builtin_nontemporal_load((const v4i*)(wsrc[s] + k * 128));               // rows 0..7
            whi[p][s] = __builtin_nontemporal_load((const v4i*)(wsrc[s] + wrow8[s] + k * 128));    // rows 8..15
        }
    };
    // RING: lane offsets of its two rows from b (< 2^32) and the wavefront-uniform address of its first K block
    static_assert(!RING || (S == 1 && NPF == 8), "the ring variant is written for one strip and eight slots");
    const uint32_t ring_lo = (uint32_t)min(n0 + (fr & 7), N - 1) * (uint32_t)K + (fr >> 3) * 64 + fq * 16;
    const uint32_t ring_hi = (uint32_t)min(n0 + (fr & 7) + 8, N - 1) * (uint32_t)K + (fr >> 3) * 64 + fq * 16;
    const uint8_t* ring_base = b + (size_t)kb0 * 128;
#define DSV3_FETCH(P_, BASE_) { DSV3_GLOAD(wlo[P_][0], ring_lo, BASE_, P_ * 128); DSV3_GLOAD(whi[P_][0], ring_hi, BASE_, P_ * 128); }
    if constexpr (RING) {
        DSV3_FETCH(0, ring_base) DSV3_FETCH(1, ring_base) DSV3_FETCH(2, ring_base) DSV3_FETCH(3, ring_base)
        DSV3_FETCH(4, ring_base) DSV3_FETCH(5, ring_base) DSV3_FETCH(6, ring_base) DSV3_FETCH(7, ring_base)
    } else {
#pragma unroll
        for (int p = 0; p < NPF; ++p)
            if (p < nkb) fetch(p, p);
    }
    if (QF) {
        // the 8 lanes that hold the chunks of one (row, K block) are consecutive and aligned: amax by DPP
#pragma unroll
        for (int i = 0; i < kSlabChunks; ++i) {
            // (the 16 values are widened twice, for the maximum and for the quotients, instead of being kept: with the
            // weight ring live this section must stay inside the register budget)
            auto widen = [&](int e) { return (e & 1) ? bf16hi_to_f32(raw[i][e >> 3][(e >> 1) & 3]) : bf16lo_to_f32(raw[i][e >> 3][(e >> 1) & 3]); };
            // largest |x| as a bit pattern (non-finite values reach the scale as in act_quant), two bf16 patterns per
            // instruction: the sixteen values are not widened for it
            uint32_t m2 = 0u;
#pragma unroll
            for (int e = 0; e < 8; ++e) m2 = pk_umax_u16(m2, raw[i][e >> 2][e & 3] & 0x7fff7fffu);
            uint32_t abits = umax_u32(m2 & 0xffffu, m2 >> 16) << 16;
            abits = dpp_umax<0xB1>(abits);       // quad_perm [1,0,3,2]
            abits = dpp_umax<0x4E>(abits);       // quad_perm [2,3,0,1]
            abits = dpp_umax<0x141>(abits);      // row_half_mirror
            const float sc = block_scale(abits, ue8m0 != 0);
            const bool fast = block_is_finite(abits);
            const float r = 1.0f / sc;
            v4i o;
            // x / sc, correctly rounded for bf16 x with |x| <= amax (as act_quant).  In a block with a non-finite value
            // the quotient needs no division either: sc = inf gives r = 0 and x * 0 is the IEEE x / inf (+-0 for finite
            // x, NaN for infinite x), sc = NaN gives NaN; only the correction step must be left out there.
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float q[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x = widen(4 * g + e), q0 = x * r;
                    q[e] = fast ? block_quotient(x, sc, r, true) : q0;
                }
                o[g] = (int)pack_fp8x4(q[0], q[1], q[2], q[3]);
            }
            const int c = tid + i * (int)blockDim.x;
            if (c < chunks) {
                const int ch = c & 7, R = c >> 3;
                *(v4i*)(act + R * 128 + ((ch ^ swz(R)) * 16)) = o;
                if (ch == 0) act_s[R] = sc * stage_q[i];
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < kSlabChunks; ++i) {
            const int c = tid + i * (int)blockDim.x;
            if (c < chunks) {
                const int ch = c & 7, R = c >> 3;
                *(v4i*)(act + R * 128 + ((ch ^ swz(R)) * 16)) = stage[i];
            }
        }
        if (tid < wg_nkb * M) act_s[tid] = stage_sa * stage_sb;
    }
    __syncthreads();

    v4f acc[S][MT];
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[s][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    // a lane's fragment: slab row (K block)*M + 16j + fr, logical chunks fq and 4 + fq of the K block
    const int row0 = (kb0 - wg_kb0) * M + fr;

    // one K block k of the wavefront's range: ring slot p holds its weights
    auto consume = [&](int p, int k) {
        v8i af[MT], wf[S];
        float sc[MT];
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int R = row0 + k * M + j * 16, fx = swz(R);
            const uint8_t* r = act + R * 128;
            af[j] = join(*(const v4i*)(r + ((fq ^ fx) * 16)), *(const v4i*)(r + (((4 + fq) ^ fx) * 16)));
            sc[j] = act_s[R];
        }
#pragma unroll
        for (int s = 0; s < S; ++s) wf[s] = untangle(wlo[p][s], whi[p][s]);
#pragma unroll
        for (int s = 0; s < S; ++s)
#pragma unroll
            for (int j = 0; j < MT; ++j) {
                const v4f z = {0.f, 0.f, 0.f, 0.f};
                const v4f p4 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[s], af[j], z, 0, 0, 0, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[s][j][e] = __builtin_fmaf(p4[e], sc[j], acc[s][j][e]);
            }
    };
    if constexpr (RING) {
        const int rounds = nkb / NPF;
        int k = 0;
        for (int r = 0; r + 1 < rounds; ++r) {              // steady state: every slot is refilled after use
            const uint8_t* nbase = ring_base + (size_t)(r + 1) * NPF * 128;       // the K blocks one ring ahead
#define DSV3_STEADY(P_) { WaitFor<2 * (NPF - 1)>::on(wlo[P_][0], whi[P_][0]); consume(P_, k); ++k; DSV3_FETCH(P_, nbase) }
            DSV3_STEADY(0) DSV3_STEADY(1) DSV3_STEADY(2) DSV3_STEADY(3) DSV3_STEADY(4) DSV3_STEADY(5) DSV3_STEADY(6) DSV3_STEADY(7)
#undef DSV3_STEADY
        }
#define DSV3_DRAIN(P_) { WaitFor<2 * (NPF - 1 - P_)>::on(wlo[P_][0], whi[P_][0]); consume(P_, k); ++k; }
        DSV3_DRAIN(0) DSV3_DRAIN(1) DSV3_DRAIN(2) DSV3_DRAIN(3) DSV3_DRAIN(4) DSV3_DRAIN(5) DSV3_DRAIN(6) DSV3_DRAIN(7)
#undef DSV3_DRAIN
    } else {
        // The wavefront works through its K blocks in batches of NPF: all weight loads of a batch are issued back
        // to back, then consumed in order.  Memory-level parallelism across batches comes from the other wavefronts
        // of the CU (up to 16), which are at different points of their own batches.
        for (int kb = 0; kb < nkb; kb += NPF) {
            if (kb > 0) {
#pragma unroll
                for (int p = 0; p < NPF; ++p)
                    if (kb + p < nkb) fetch(p, kb + p);
            }
#pragma unroll
            for (int p = 0; p < NPF; ++p)
                if (kb + p < nkb) consume(p, kb + p);             // wavefront-uniform
        }
    }
#undef DSV3_FETCH
    __syncthreads();                                        // everyone is done with the activation slab

    // ---- add the wavefronts' partial sums in LDS (fixed order), then store
    v4f* red = (v4f*)lds;                                   // [wave][s*MT + j][lane]
    constexpr int TILES = S * MT;
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int j = 0; j < MT; ++j) red[(wave * TILES + s * MT + j) * 64 + lane] = acc[s][j];
    __syncthreads();
    const size_t slab = (size_t)blockIdx.y * M * N;          // split-K slab of the fp32 workspace (0 when gridDim.y == 1)
    for (int slot = tid; slot < TILES * 64; slot += blockDim.x) {
        // the partial sums of the wavefronts, added in wavefront order; read four at a time so that the LDS latency
        // is paid once per four and not once per wavefront (a missing wavefront re-reads the last one, weight 0)
        v4f v = red[slot];
        for (int w0 = 1; w0 < n_waves; w0 += 4) {
            v4f u[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) u[i] = red[min(w0 + i, n_waves - 1) * TILES * 64 + slot];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (w0 + i < n_waves) { v[0] += u[i][0]; v[1] += u[i][1]; v[2] += u[i][2]; v[3] += u[i][3]; }
            }
        }
        const int t = slot >> 6, l = slot & 63;
        const int s = t / MT, j = t % MT;
        const int m = j * 16 + (l & 15);
        const int n = n0 + s * 16 + (l >> 4) * 4;
        if (m >= M) continue;
        const size_t idx = slab + (size_t)m * N + n;
        if (n + 3 < N && (N & 3) == 0) {                      // four results in one store
            if (out_dtype == DSV3_F32) *(v4f*)((float*)out + idx) = v;
            else if (out_dtype == DSV3_BF16) *(v2u*)((uint16_t*)out + idx) = v2u{ pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]) };
            else *(v2u*)((uint16_t*)out + idx) = v2u{ pack_f16(v[0], v[1]), pack_f16(v[2], v[3]) };
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e >= N) break;
            if (out_dtype == DSV3_F32)       ((float*)out)[idx + e] = v[e];
            else if (out_dtype == DSV3_BF16) ((uint16_t*)out)[idx + e] = cvt_out<DSV3_BF16>(v[e]);
            else                             ((uint16_t*)out)[idx + e] = cvt_out<DSV3_F16>(v[e]);
        }
    }
}

struct Plan { int mt, s, waves, splits, kb_per_wg; };

// The kernels here run for 5-30 us, so the grid is sized to be resident in ONE round: the workgroups of a
// second, partly filled round would leave most of the chip idle for half the run.  Within that limit: as many
// wavefronts as possible (memory-level parallelism), at least two K blocks per wavefront, and few K splits
// across workgroups (each costs an [M,N] fp32 slab of traffic plus the reduction pass).
inline Plan make_plan(int64_t m, int64_t n, int64_t k) {
    const int64_t kb = k / 128;
    const int64_t capacity = 256 * 16;                         // resident wavefronts: 256 CUs x 16 (<= 128 VGPRs)
    Plan best{};
    bool have = false;
    // wider strips per wavefront (S) cut the number of workgroups when the activation slab forces many K splits
    for (int s_ : {1, 2, 4}) {
        Plan p;
        p.mt = 1;
        p.s = s_;
        const int64_t groups = (n + 16 * s_ - 1) / (16 * s_);
        // more wavefronts per workgroup = fewer K splits, down to a single pass: at one row 16 against 4 gives
        // wq_a 7168 -> 1536 8.05 -> 6.8 us, wo 16384 -> 7168 27.0 -> 25.6 us; from a few rows up the activation slab a
        // workgroup stages first grows with its K range, and 8 is the better limit (wkv_a at 8 rows: 7.2 against 7.8 us)
        int waves = m <= 2 ? kMaxWaves : 8;
        while (waves > 1 && (kb / waves < 2 || groups * waves > capacity)) waves >>= 1;
        int64_t splits = capacity / (groups * waves);
        const int64_t max_splits = kb / (2 * waves) > 0 ? kb / (2 * waves) : 1;
        if (splits > max_splits) splits = max_splits;
        // the activation slab (m rows x 128 B per K block) is staged through kSlabChunks registers per thread,
        // and one scale per thread
        int64_t slab_kb = (int64_t)kSlabChunks * waves * 64 / (m * 8);
        if (slab_kb > waves * 64 / m) slab_kb = waves * 64 / m;
        if (slab_kb > 480 / m) slab_kb = 480 / m;              // (slab_kb m + 16) 128 + 4 slab_kb m <= 64 KiB of LDS
        if (slab_kb < 1) continue;
        const int64_t min_splits = (kb + slab_kb - 1) / slab_kb;
        if (splits < min_splits) splits = min_splits;
        if (splits < 1) splits = 1;
        p.waves = waves;
        p.kb_per_wg = (int)((kb + splits - 1) / splits);
        p.splits = (int)((kb + p.kb_per_wg - 1) / p.kb_per_wg);
        const bool fits = groups * p.splits * waves <= capacity;
        if (!have || fits) { best = p; have = true; }
        if (fits) break;
    }
    return best;
}

template <int MT, int S, bool QF>
void launch_cfg(const Plan& p, const void* a, const float* a_s, const void* b, const float* b_s,
                void* out, int out_dtype, int m, int n, int k, int ue8m0, hipStream_t st) {
    constexpr int NPF = 8 / S;
    const unsigned groups = (unsigned)((n + 16 * S - 1) / (16 * S));
    const size_t red_bytes = (size_t)p.waves * S * MT * 64 * sizeof(v4f);
    const size_t slab_bytes = ((size_t)p.kb_per_wg * m + 16) * 128 + (size_t)p.kb_per_wg * m * 4;
    const size_t lds = red_bytes > slab_bytes ? red_bytes : slab_bytes;
    const uint64_t m_magic = (uint64_t)(((1ull << 32) + (uint64_t)m - 1) / (uint64_t)m);
    if constexpr (S == 1) {
        // every wavefront's K range: the same whole number (>= 2) of ring rounds
        const int kb = k / 128, per_wave = p.kb_per_wg / p.waves;
        static const bool no_ring = getenv("DSV3_SKINNY_NORING") != nullptr;
        if (!no_ring && kb % p.kb_per_wg == 0 && p.kb_per_wg % p.waves == 0 && per_wave % NPF == 0 && per_wave >= 2 * NPF &&
            (int64_t)n * k < (1ll << 32)) {
            hipLaunchKernelGGL((fp8_gemm_skinny_kernel<MT, S, NPF, QF, true>), dim3(groups, (unsigned)p.splits), dim3(p.waves * kWave), lds, st,
                               (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, out, out_dtype, m, n, k, p.kb_per_wg, ue8m0, m_magic);
            return;
        }
    }
    hipLaunchKernelGGL((fp8_gemm_skinny_kernel<MT, S, NPF, QF>), dim3(groups, (unsigned)p.splits), dim3(p.waves * kWave), lds, st,
                       (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, out, out_dtype, m, n, k, p.kb_per_wg, ue8m0, m_magic);
}

}  // namespace skinny

bool skinny_supported(int64_t m, int64_t n, int64_t k) {
    return m >= 1 && m <= 16 && k >= 128 && n >= 1 && (n + 15) / 16 <= 0x7fffffff;
}

size_t skinny_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    const skinny::Plan p = skinny::make_plan(m, n, k);
    return p.splits > 1 ? (size_t)p.splits * (size_t)m * (size_t)n * sizeof(float) : 0;
}

// Runs the streaming kernel; *splits_out tells the caller how many fp32 slabs were written to `ws`
// (1 = the result went straight to c).  quant_mode 0: a is fp8 with scales a_s; 1 / 2: a is bf16 and is quantised
// inside the kernel (scale_fmt none / ue8m0).
int launch_skinny(const void* a, const float* a_s, const void* b, const float* b_s, void* c, int c_dtype,
                  int64_t m, int64_t n, int64_t k, void* ws, int* splits_out, hipStream_t st, int quant_mode) {
    using namespace skinny;
    const Plan p = make_plan(m, n, k);
    void* out = p.splits > 1 ? ws : c;
    const int od = p.splits > 1 ? (int)DSV3_F32 : c_dtype;
    *splits_out = p.splits;
    const int ue = quant_mode == 2;
#define DSV3_CASE(MT_, S_)                                                                                   \
    if (quant_mode) launch_cfg<MT_, S_, true>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, ue, st);  \
    else launch_cfg<MT_, S_, false>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, 0, st);             \
    break
    switch (p.mt * 10 + p.s) {
        case 11: DSV3_CASE(1, 1);
        case 12: DSV3_CASE(1, 2);
        case 14: DSV3_CASE(1, 4);
        default: return DSV3_ERR_BAD_SHAPE;
    }
#undef DSV3_CASE
    return launch_status();
}

}  // namespace dsv3
