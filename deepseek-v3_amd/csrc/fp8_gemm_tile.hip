// fp8_gemm, large-M kernel for gfx950 (reference: inference/kernel.py:118-172).
//
//   c[m,n] = sum_kb ( sum_{t<128} a[m,128kb+t] * b[n,128kb+t] ) * a_s[m,kb] * b_s[n/128,kb]
//
// A workgroup owns a BM x BN tile of C and walks K in blocks of 128 -- exactly
// one scale block -- staging the A rows and the B rows (both K-contiguous) in
// LDS, double buffered.  Each wavefront computes a WM x WN sub-tile out of
// 16x16 MFMA tiles with v_mfma_f32_16x16x128_f8f6f4: one instruction consumes a
// whole scale block of K and returns its raw dot products, which are folded into
// the binary32 accumulators with one FMA each by the block's scale.
//
// The MFMA is issued "transposed": the weight rows (n) are the instruction's A
// operand and the activation rows (m) its B operand, so a lane's four results
// share one m.  That makes the scale a single value per lane and 16-row
// sub-tile ( a_s[m,kb] * b_s[n/128,kb] with the b_s factor uniform over the
// workgroup because BN divides 128-aligned tiles ), and it makes a lane's four
// results consecutive in n for the store.
//
// Both operands take their 32 bytes per lane from the same K offsets, so the
// result does not depend on how the instruction numbers K internally.
#include "common.hpp"
#include <cstdlib>
#include <cstring>

namespace dsv3 {
namespace {

constexpr int kRowStride = 128 + 16;     // padded: consecutive rows land in different banks

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    v8i r = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
    return r;
}

template <int BM, int BN, int WM, int WN, int CD>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave, 2) void fp8_gemm_tile_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c,
        int M, int N, int K, int tiles_m, int tiles_n, int kb_per_split) {
    constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    constexpr int THREADS = WAVES_M * WAVES_N * kWave;
    constexpr int SM = WM / 16, SN = WN / 16;             // 16x16 sub-tiles per wave
    constexpr int A_CHUNKS = BM * 8 / THREADS;            // 16-byte chunks a thread stages per K block
    constexpr int B_CHUNKS = BN * 8 / THREADS;
    constexpr int STAGE = (BM + BN) * kRowStride;
    static_assert(BM * 8 % THREADS == 0 && BN * 8 % THREADS == 0, "tile/threads mismatch");
    static_assert(BN <= 128 && 128 % BN == 0, "b_s must be uniform over the tile");

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // ---- workgroup -> tile: give each XCD (workgroups are dealt round-robin to the 8 XCDs)
    // a contiguous run of tiles, and walk tiles in bands of GROUP_M tile-rows for L2 reuse.
    const int T = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int q = T / 8, r = T % 8, x = pid % 8;
        pid = x * q + (x < r ? x : r) + pid / 8;
    }
    constexpr int GROUP_M = 8;
    const int band = pid / (GROUP_M * tiles_n);
    const int band_rows = min(GROUP_M, tiles_m - band * GROUP_M);
    const int in_band = pid - band * GROUP_M * tiles_n;
    const int tm = band * GROUP_M + in_band % band_rows;
    const int tn = in_band / band_rows;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int KB = K / 128;                       // row stride of both scale tensors
    // split-K: blockIdx.y owns K blocks [kb0, kb0 + nkb) and writes its own [M,N] slab of c
    const int kb0 = blockIdx.y * kb_per_split;
    const int nkb = min(kb_per_split, KB - kb0);
    c += (size_t)blockIdx.y * M * N;

    // ---- global -> register staging: chunk id = i*THREADS + tid -> (row = id/8, chunk = id%8)
    const uint8_t* a_src[A_CHUNKS];
    const uint8_t* b_src[B_CHUNKS];
    int a_dst[A_CHUNKS], b_dst[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int id = i * THREADS + tid, row = id >> 3, ch = id & 7;
        a_src[i] = a + (size_t)min(m0 + row, M - 1) * K + kb0 * 128 + ch * 16;
        a_dst[i] = row * kRowStride + ch * 16;
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
        const int id = i * THREADS + tid, row = id >> 3, ch = id & 7;
        b_src[i] = b + (size_t)min(n0 + row, N - 1) * K + kb0 * 128 + ch * 16;
        b_dst[i] = BM * kRowStride + row * kRowStride + ch * 16;
    }

    // ---- per-lane scale sources: a_s[m, kb] for the lane's row of each 16-row sub-tile
    const float* as_src[SM];
#pragma unroll
    for (int j = 0; j < SM; ++j)
        as_src[j] = a_s + (size_t)min(m0 + wm * WM + j * 16 + (lane & 15), M - 1) * KB + kb0;
    const float* bs_src = b_s + (size_t)(n0 / 128) * KB + kb0;

    // ---- LDS read offsets of the lane's 32 bytes inside a tile row
    const int frag_off = (lane & 15) * kRowStride + (lane >> 4) * 32;
    const int a_rd = wm * WM * kRowStride + frag_off;
    const int b_rd = BM * kRowStride + wn * WN * kRowStride + frag_off;

    v4f acc[SN][SM];
#pragma unroll
    for (int i = 0; i < SN; ++i)
#pragma unroll
        for (int j = 0; j < SM; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    v4i a_st[A_CHUNKS], b_st[B_CHUNKS];
    float as_cur[SM], as_nxt[SM];
    float bs_cur, bs_nxt = 0.f;

    // prologue: K block 0 -> LDS stage 0
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) a_st[i] = *(const v4i*)(a_src[i]);
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) b_st[i] = *(const v4i*)(b_src[i]);
#pragma unroll
    for (int j = 0; j < SM; ++j) as_cur[j] = as_src[j][0];
    bs_cur = bs_src[0];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) *(v4i*)(lds + a_dst[i]) = a_st[i];
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) *(v4i*)(lds + b_dst[i]) = b_st[i];
    __syncthreads();

    for (int kb = 0; kb < nkb; ++kb) {
        const uint8_t* cur = lds + (kb & 1) * STAGE;
        uint8_t* nxt = lds + ((kb + 1) & 1) * STAGE;
        const bool more = kb + 1 < nkb;
        if (more) {
            const int ko = (kb + 1) * 128;
#pragma unroll
            for (int i = 0; i < A_CHUNKS; ++i) a_st[i] = *(const v4i*)(a_src[i] + ko);
#pragma unroll
            for (int i = 0; i < B_CHUNKS; ++i) b_st[i] = *(const v4i*)(b_src[i] + ko);
#pragma unroll
            for (int j = 0; j < SM; ++j) as_nxt[j] = as_src[j][kb + 1];
            bs_nxt = bs_src[kb + 1];
        }

        v8i af[SM];
#pragma unroll
        for (int j = 0; j < SM; ++j) {
            const uint8_t* p = cur + a_rd + j * 16 * kRowStride;
            af[j] = join(*(const v4i*)p, *(const v4i*)(p + 16));
        }
        float sc[SM];
#pragma unroll
        for (int j = 0; j < SM; ++j) sc[j] = as_cur[j] * bs_cur;
#pragma unroll
        for (int i = 0; i < SN; ++i) {
            const uint8_t* p = cur + b_rd + i * 16 * kRowStride;
            const v8i bf = join(*(const v4i*)p, *(const v4i*)(p + 16));
#pragma unroll
            for (int j = 0; j < SM; ++j) {
                const v4f z = {0.f, 0.f, 0.f, 0.f};
                const v4f p4 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af[j], z, 0, 0, 0, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][e] = __builtin_fmaf(p4[e], sc[j], acc[i][j][e]);
            }
        }

        if (more) {
#pragma unroll
            for (int i = 0; i < A_CHUNKS; ++i) *(v4i*)(nxt + a_dst[i]) = a_st[i];
#pragma unroll
            for (int i = 0; i < B_CHUNKS; ++i) *(v4i*)(nxt + b_dst[i]) = b_st[i];
#pragma unroll
            for (int j = 0; j < SM; ++j) as_cur[j] = as_nxt[j];
            bs_cur = bs_nxt;
        }
        __syncthreads();
    }

    // ---- epilogue: lane holds c[m][n .. n+3] per sub-tile
    const bool vec_ok = (N % 4) == 0;
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        const int m = m0 + wm * WM + j * 16 + (lane & 15);
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < SN; ++i) {
            const int n = n0 + wn * WN + i * 16 + (lane >> 4) * 4;
            typename OutT<CD>::type* dst = c + (size_t)m * N + n;
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

// Sums the split-K slabs in a fixed order (slab 0 first) and converts to the output type.  A thread owns four
// consecutive outputs and requests eight slabs' worth of partial sums before it adds the first: written as a loop of
// load-then-add, every slab cost a round trip to L2 (0.6-0.8 us each on the decode shapes, measured).  Slabs past the
// last one are requested again from the last slab and left out of the sum (no "+ 0": a sum that is -0 stays -0).
template <int CD>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(
        const float* __restrict__ ws, typename OutT<CD>::type* __restrict__ c, int64_t mn, int splits) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= mn) return;
    constexpr int U = 8;
    if ((mn & 3) == 0) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < splits; s += U) {
            v4f t[U];
#pragma unroll
            for (int u = 0; u < U; ++u) t[u] = *(const v4f*)(ws + (int64_t)min(s + u, splits - 1) * mn + i);
#pragma unroll
            for (int u = 0; u < U; ++u) v = s + u < splits ? v + t[u] : v;
        }
        if (CD == DSV3_F32) *(v4f*)(c + i) = v;
        else if (CD == DSV3_BF16) *(v2u*)(c + i) = v2u{ pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]) };
        else *(v2u*)(c + i) = v2u{ pack_f16(v[0], v[1]), pack_f16(v[2], v[3]) };
        return;
    }
    const int64_t left = mn - i;                    // 1 .. 4 outputs when mn is not a multiple of four
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < splits; s += U) {
        float t[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) t[u][e] = ws[(int64_t)min(s + u, splits - 1) * mn + i + (e < left ? e : 0)];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = s + u < splits ? v[e] + t[u][e] : v[e];
    }
    for (int e = 0; e < 4 && e < left; ++e) c[i + e] = cvt_out<CD>(v[e]);
}
inline unsigned splitk_reduce_grid(int64_t mn) { return (unsigned)(((mn + 3) / 4 + 255) / 256); }

template <int BM, int BN, int WM, int WN, int CD>
int launch_cfg(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
               int64_t m, int64_t n, int64_t k, int splits, int kb_per_split, hipStream_t stream) {
    const int64_t tm = (m + BM - 1) / BM, tn = (n + BN - 1) / BN;
    if (tm * tn > 0x7fffffff || splits > 65535) return DSV3_ERR_BAD_SHAPE;
    auto kern = fp8_gemm_tile_kernel<BM, BN, WM, WN, CD>;
    constexpr int lds_bytes = 2 * (BM + BN) * kRowStride;
    static LdsGrant grant;                   // more than the default 64 KiB of dynamic LDS
    if (!grant.ensure((const void*)kern, lds_bytes)) return DSV3_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tm * tn), (unsigned)splits), dim3((BM / WM) * (BN / WN) * kWave), lds_bytes, stream,
                       (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, (typename OutT<CD>::type*)c,
                       (int)m, (int)n, (int)k, (int)tm, (int)tn, kb_per_split);
    return launch_status();
}

// Split-K plan for skinny problems: enough workgroups to cover the chip a few times over,
// but at least 4 K blocks per split.
struct Plan { int bm; int splits; int kb_per_split; };

Plan make_plan(int64_t m, int64_t n, int64_t k) {
    Plan p;
    p.bm = m <= 32 ? 32 : (m <= 64 ? 64 : 128);
    const int64_t kb = k / 128;
    p.splits = 1;
    p.kb_per_split = (int)kb;
    if (m <= 64 && kb > 0) {
        const int64_t tiles = (n + 127) / 128;
        const int64_t target = 1024;                       // workgroups wanted (256 CUs x 4)
        int64_t s = (target + tiles - 1) / tiles;
        int64_t max_s = kb / 4 > 0 ? kb / 4 : 1;
        if (s > max_s) s = max_s;
        if (s < 1) s = 1;
        p.kb_per_split = (int)((kb + s - 1) / s);
        p.splits = (int)((kb + p.kb_per_split - 1) / p.kb_per_split);
    }
    return p;
}

// K not a multiple of 128 (inference/kernel.py:145, 158-159: the reference's kernel masks the last, partial K block;
// its act_quant cannot produce such an operand, kernel.py:52, so nothing on the model's path gets here).  A plain
// kernel for completeness, not for speed: rows of a and b are not 16-byte aligned then, so everything is read bytewise.
// One thread per output element; a workgroup owns one row of a and 256 columns, stages the row's K block in LDS as
// binary32 and walks the K blocks in the reference's order: (dot * a_s) * b_s, accumulated in binary32.  The scale
// tensors have ceil(K / 128) columns.
template <int CD>
__global__ __launch_bounds__(256) void fp8_gemm_any_k_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        typename OutT<CD>::type* __restrict__ c, int M, int N, int K) {
    __shared__ float arow[128];
    const int m = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    const int KB = (K + 127) / 128;
    const uint8_t* brow = b + (size_t)min(n, N - 1) * K;
    float acc = 0.f;
    for (int kb = 0; kb < KB; ++kb) {
        const int len = min(128, K - kb * 128);
        __syncthreads();
        if ((int)threadIdx.x < len)
            arow[threadIdx.x] = __builtin_amdgcn_cvt_f32_fp8((int)a[(size_t)m * K + kb * 128 + threadIdx.x], 0);
        __syncthreads();
        float dot = 0.f;
        for (int t = 0; t < len; ++t)
            dot = __builtin_fmaf(arow[t], __builtin_amdgcn_cvt_f32_fp8((int)brow[kb * 128 + t], 0), dot);
        acc += (dot * a_s[(size_t)m * KB + kb]) * b_s[(size_t)(min(n, N - 1) / 128) * KB + kb];
    }
    if (n < N) c[(size_t)m * N + n] = cvt_out<CD>(acc);
}

// 3 to 16 rows on a weight of 96 MiB or more for which the activation-streaming kernel has no plan: the dense GEMM runs
// as one group of the grouped weight-streaming kernel -- 32-row strips of such a weight fill the chip, one launch, no
// partial sums in memory.
bool single_group_stream(int64_t m, int64_t n, int64_t k) {
    if (m < 3 || m > 16 || n * k < (96ll << 20) || !skinny_single_supported(m, n, k)) return false;
    // wherever the activation-streaming kernel has a plan it is faster (16384 -> 7168 at 4 / 8 / 16 rows: 22.2 / 22.5 /
    // 23.5 against 25.6 / 26.7 / 29.6 us; 7168 -> 18432: 22 / 22 / 22.8 against 28.5 / 31 / 36.5 us)
    return !stream_supported(m, n, k);
}

// DSV3_GEMM_FORCE=tile|prefill|stream|skinny pins the kernel choice where the named kernel supports the shape (tuning /
// debugging aid).
int forced_kernel() {
    static const int v = [] {
        const char* e = std::getenv("DSV3_GEMM_FORCE");
        if (!e) return 0;
        if (!std::strcmp(e, "tile")) return 1;
        if (!std::strcmp(e, "prefill")) return 2;
        if (!std::strcmp(e, "stream")) return 3;
        if (!std::strcmp(e, "skinny")) return 4;
        return 0;
    }();
    return v;
}

// Which problems go to the large-M kernel (K range cut into slices when the tiles do not fill the chip): every M
// above 64, and M = 33 .. 64 when the weight is large (>= 96 MiB) and has 8192 rows or more (7168 -> 36864 at 64 rows:
// 65 against 66-76 us).  There it runs at a flat 32-34 us per 117-132 MB from 9 to 64 rows.  Everything else the
// activation-streaming kernel has a plan for goes there (16384 -> 7168 at 16 / 32 / 64 rows 23.5 / 24.5 / 29.5 against
// 33 / 31.6 / 34.6 us; 7168 -> 18432 at 16 / 32 rows 22.8 / 25.3 against 36.5 / 30.7 us); for the smaller decode
// weights the streaming and tile kernels are faster anyway.
bool to_large_m_kernel(int64_t m, int64_t n, int64_t k) {
    if (!prefill_supported(m, n, k)) return false;
    if (m > 64) return true;
    if (m <= 8 || n * k < (96ll << 20)) return false;
    return !((n < 8192 || m <= 32) && stream_supported(m, n, k));
}

template <int CD>
int launch_typed(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                 int64_t m, int64_t n, int64_t k, void* ws, hipStream_t st, bool pow2) {
    if (k == 0) {   // empty sum: c = 0
        const int64_t mn0 = m * n;
        hipLaunchKernelGGL((splitk_reduce_kernel<CD>), dim3(splitk_reduce_grid(mn0)), dim3(256), 0, st,
                           (const float*)nullptr, (typename OutT<CD>::type*)c, mn0, 0);
        return launch_status();
    }
    if (k % 128 != 0) {
        hipLaunchKernelGGL((fp8_gemm_any_k_kernel<CD>), dim3((unsigned)((n + 255) / 256), (unsigned)m), dim3(256), 0, st,
                           (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, (typename OutT<CD>::type*)c, (int)m, (int)n, (int)k);
        return launch_status();
    }
    const int force = forced_kernel();
    if (force == 0 && single_group_stream(m, n, k))
        return launch_skinny_single(a, a_s, b, b_s, c, CD, m, n, k, st);
    const bool to_prefill = force != 1 && !(force == 3 && stream_supported(m, n, k)) && to_large_m_kernel(m, n, k);
    const bool use_stream = force != 1 && !to_prefill && !(force == 4 && skinny_supported(m, n, k)) && stream_supported(m, n, k);
    if (use_stream || (force != 1 && !to_prefill && skinny_supported(m, n, k))) {          // decode shapes: weight-streaming kernels
        int splits = 1;
        const int rc = use_stream ? launch_stream(a, a_s, b, b_s, c, CD, m, n, k, ws, &splits, st)
                                  : launch_skinny(a, a_s, b, b_s, c, CD, m, n, k, ws, &splits, st);
        if (rc != DSV3_OK || splits == 1) return rc;
        const int64_t mn = m * n;
        hipLaunchKernelGGL((splitk_reduce_kernel<CD>), dim3(splitk_reduce_grid(mn)), dim3(256), 0, st,
                           (const float*)ws, (typename OutT<CD>::type*)c, mn, splits);
        return launch_status();
    }
    if (to_prefill) return pow2 ? launch_prefill<CD, true>(a, a_s, b, b_s, c, m, n, k, ws, st)
                                : launch_prefill<CD, false>(a, a_s, b, b_s, c, m, n, k, ws, st);
    const Plan p = make_plan(m, n, k);
    if (p.splits == 1) {
        if (p.bm == 32) return launch_cfg<32, 128, 32, 32, CD>(a, a_s, b, b_s, c, m, n, k, 1, p.kb_per_split, st);
        if (p.bm == 64) return launch_cfg<64, 128, 64, 32, CD>(a, a_s, b, b_s, c, m, n, k, 1, p.kb_per_split, st);
        return launch_cfg<128, 128, 64, 64, CD>(a, a_s, b, b_s, c, m, n, k, 1, p.kb_per_split, st);
    }
    int rc;
    if (p.bm == 32) rc = launch_cfg<32, 128, 32, 32, DSV3_F32>(a, a_s, b, b_s, ws, m, n, k, p.splits, p.kb_per_split, st);
    else            rc = launch_cfg<64, 128, 64, 32, DSV3_F32>(a, a_s, b, b_s, ws, m, n, k, p.splits, p.kb_per_split, st);
    if (rc != DSV3_OK) return rc;
    const int64_t mn = m * n;
    hipLaunchKernelGGL((splitk_reduce_kernel<CD>), dim3(splitk_reduce_grid(mn)), dim3(256), 0, st,
                       (const float*)ws, (typename OutT<CD>::type*)c, mn, p.splits);
    return launch_status();
}

}  // namespace

// linear() of the reference for few rows (inference/model.py:159-160: act_quant, then fp8_gemm) as ONE launch:
// the M <= 16 weight-streaming kernel quantises the bf16 activations itself.  Same workspace as fp8_gemm.
// Every workgroup quantises the rows of its own K range again, so the fusion pays while the activation matrix is
// small (16 rows x 16384: 51 us fused against 44 us in two launches; 8 rows: equal; fewer: 1 - 3 us saved).  Shapes
// that fp8_gemm itself sends to another kernel (3+ rows on long K ranges: the activation-streaming kernel) are not
// fused, so that the one call and the two calls always give the same bits.
bool linear_fp8_supported(int64_t m, int64_t n, int64_t k) {
    return forced_kernel() != 1 && k % 128 == 0 && skinny_supported(m, n, k) && !to_large_m_kernel(m, n, k) &&
           !(forced_kernel() == 0 && single_group_stream(m, n, k)) && (m <= 2 || !stream_supported(m, n, k)) &&
           m * k <= 131072;
}

int launch_linear_fp8(const void* x, const void* b, const float* b_s, void* c, int c_dtype, int64_t m, int64_t n,
                      int64_t k, int scale_fmt, void* ws, hipStream_t st) {
    int splits = 1;
    const int rc = launch_skinny(x, nullptr, b, b_s, c, c_dtype, m, n, k, ws, &splits, st,
                                 scale_fmt == DSV3_SCALE_FMT_UE8M0 ? 2 : 1);
    if (rc != DSV3_OK || splits == 1) return rc;
    const int64_t mn = m * n;
    switch (c_dtype) {
        case DSV3_BF16: hipLaunchKernelGGL((splitk_reduce_kernel<DSV3_BF16>), dim3(splitk_reduce_grid(mn)), dim3(256), 0, st, (const float*)ws, (uint16_t*)c, mn, splits); break;
        case DSV3_F16:  hipLaunchKernelGGL((splitk_reduce_kernel<DSV3_F16>), dim3(splitk_reduce_grid(mn)), dim3(256), 0, st, (const float*)ws, (uint16_t*)c, mn, splits); break;
        default:        hipLaunchKernelGGL((splitk_reduce_kernel<DSV3_F32>), dim3(splitk_reduce_grid(mn)), dim3(256), 0, st, (const float*)ws, (float*)c, mn, splits); break;
    }
    return launch_status();
}

size_t fp8_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const Plan p = make_plan(m, n, k);
    const size_t tile_ws = p.splits > 1 ? (size_t)p.splits * (size_t)m * (size_t)n * sizeof(float) : 0;
    size_t need = tile_ws;
    if (skinny_supported(m, n, k) && skinny_workspace_bytes(m, n, k) > need) need = skinny_workspace_bytes(m, n, k);
    if (stream_supported(m, n, k) && stream_workspace_bytes(m, n, k) > need) need = stream_workspace_bytes(m, n, k);
    if (to_large_m_kernel(m, n, k) && prefill_workspace_bytes(m, n, k) > need) need = prefill_workspace_bytes(m, n, k);
    return need;
}

int launch_fp8_gemm(const void* a, const float* a_s, const void* b, const float* b_s,
                    void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                    void* workspace, size_t workspace_bytes, hipStream_t stream, bool pow2_scales) {
    (void)workspace_bytes;
    switch (c_dtype) {
        case DSV3_BF16: return launch_typed<DSV3_BF16>(a, a_s, b, b_s, c, m, n, k, workspace, stream, pow2_scales);
        case DSV3_F16:  return launch_typed<DSV3_F16>(a, a_s, b, b_s, c, m, n, k, workspace, stream, pow2_scales);
        case DSV3_F32:  return launch_typed<DSV3_F32>(a, a_s, b, b_s, c, m, n, k, workspace, stream, pow2_scales);
        default: return DSV3_ERR_BAD_DTYPE;
    }
}

}  // namespace dsv3
