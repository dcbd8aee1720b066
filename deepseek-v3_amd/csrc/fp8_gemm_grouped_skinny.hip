// Grouped fp8_gemm for a handful of rows per group on gfx950: the weight-streaming counterpart of the grouped tile
// kernel, for the MoE layer at decode sizes (reference arithmetic: inference/kernel.py:145-172 applied per expert as
// in inference/model.py:684-689).
//
//   for every tile slot t with group g:  c[r, n] = sum_kb ( sum_{i<128} a[src(r), 128kb+i] * b_g[n, 128kb+i] )
//                                                   * a_s[src(r), kb] * b_s_g[n/128, kb]
//
// One token activates 8 routed experts (+ the shared one): 9 groups of ONE row each, 44 MB of weights per group.
// The tile kernel gives such a launch 9 x 16 workgroups -- half the chip -- and each of them is alone with a 1.8 MB
// weight slab behind a two-block prefetch.  Here a workgroup owns 32 weight rows of one group (two 16-row MFMA
// strips per wavefront) and its two to eight wavefronts split the K range, so the same launch has 9 x 128 x 4
// wavefronts streaming with three K blocks of loads in flight each.
//
// Weights go straight from global memory into MFMA operand registers exactly as in the dense decode kernel
// (fp8_gemm_skinny.hip: 8 rows x 128 contiguous bytes per load instruction, halves exchanged by DPP).  The
// activation rows (at most 16 per pass, L2-resident) are read from global memory as well, issued in the same
// order as the weights they meet, so no load waits behind a younger one; there is no LDS staging, hence no limit
// on K and no partial sums outside the workgroup.  The wavefronts' partial sums are added in LDS in a fixed
// order.  A slot with more than 16 rows is processed in passes of 16 (the weights are streamed again per pass:
// correct for any table, efficient for the small groups the dispatcher sends here).
#include "common.hpp"

namespace dsv3 {
namespace gskinny {

constexpr int S = 2;            // 16-row weight strips per wavefront

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    v8i r = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
    return r;
}

// a = what the lane loaded from rows 0..7 of a strip, b = from rows 8..15: first 16 bytes of the fragment =
// lane<8 ? a : ror8(b), last 16 bytes = lane<8 ? ror8(a) : b (row rotate by 8 inside each 16-lane row).
__device__ __forceinline__ v8i untangle(v4i a, v4i b) {
    v8i r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r[i]     = __builtin_amdgcn_update_dpp(a[i], b[i], 0x128, 0xf, 0xc, false);
        r[4 + i] = __builtin_amdgcn_update_dpp(b[i], a[i], 0x128, 0xf, 0x3, false);
    }
    return r;
}

template <int kWaves>
__global__ __launch_bounds__(kWaves * kWave) void fp8_gemm_grouped_skinny_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s, const int* __restrict__ a_rows,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s, void* __restrict__ c, int c_dtype,
        int N, int K, const int* __restrict__ tile_group, const int* __restrict__ tile_row0,
        const int* __restrict__ tile_rows, int64_t b_stride, int64_t bs_stride, int single_rows) {
    // K blocks of loads in flight per wavefront: three keep the kernel at 128 registers or fewer, i.e. 16 resident
    // wavefronts per compute unit (four blocks in flight and 12 wavefronts measured slower)
    constexpr int NPF = kWaves <= 8 ? 3 : 2;
    __shared__ v4f red[kWaves * S * 64];
    // without a tile table the launch is ONE group of single_rows rows: a dense GEMM with few rows
    const int slot = blockIdx.y;
    const int grp = tile_group ? tile_group[slot] : 0;
    if (grp < 0) return;                                   // uniform over the workgroup
    const int row0 = tile_group ? tile_row0[slot] : 0, rows = tile_group ? tile_rows[slot] : single_rows;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int fr = lane & 15, fq = lane >> 4;
    const int KB = K >> 7;
    const int per_wave = (KB + kWaves - 1) / kWaves;
    const int kb0 = wave * per_wave;
    const int nkb = max(0, min(per_wave, KB - kb0));
    const int n0 = blockIdx.x * (16 * S);
    b += (size_t)grp * b_stride;
    b_s += (size_t)grp * bs_stride + (size_t)min(n0 >> 7, (N - 1) >> 7) * KB + kb0;

    // weight loads: lanes with fr < 8 take the first 64 bytes of row fr & 7 of the strip, the others the last 64.
    // Offsets are 32-bit (the caller checks that a group's weights and the activations stay below 4 GiB) on top of
    // wavefront-uniform bases.
    uint32_t woff[S], wrow8[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const int r_lo = min(n0 + s * 16 + (fr & 7), N - 1), r_hi = min(n0 + s * 16 + (fr & 7) + 8, N - 1);
        woff[s] = (uint32_t)r_lo * (uint32_t)K + (uint32_t)kb0 * 128u + (fr >> 3) * 64 + fq * 16;
        wrow8[s] = (uint32_t)(r_hi - r_lo) * (uint32_t)K;
    }

    for (int pass = 0; pass < rows; pass += 16) {
        const int m_here = min(16, rows - pass);
        // activation fragment of lane (fr, fq): row fr of this pass (rows past its end repeat the last one; their
        // results are dropped), bytes {16 fq .. +15} and {64 + 16 fq .. +15} of the K block
        const int crow = row0 + pass + min(fr, m_here - 1);
        const uint32_t arow = (uint32_t)(a_rows ? a_rows[crow] : crow);
        const uint32_t aoff = arow * (uint32_t)K + (uint32_t)kb0 * 128u + fq * 16;
        const uint32_t asoff = arow * (uint32_t)KB + (uint32_t)kb0;

        v4i wlo[NPF][S], whi[NPF][S], alo[NPF], ahi[NPF];
        float sa[NPF], sb[NPF];
        auto fetch = [&](int p, int k) {
#pragma unroll
            for (int s = 0; s < S; ++s) {
                wlo[p][s] = __builtin_nontemporal_load((const v4i*)(b + woff[s] + (uint32_t)k * 128u));
                whi[p][s] = __builtin_nontemporal_load((const v4i*)(b + woff[s] + wrow8[s] + (uint32_t)k * 128u));
            }
            alo[p] = *(const v4i*)(a + aoff + (uint32_t)k * 128u);
            ahi[p] = *(const v4i*)(a + aoff + (uint32_t)k * 128u + 64u);
            sa[p] = a_s[asoff + (uint32_t)k];
            sb[p] = b_s[k];
        };
        v4f acc[S];
#pragma unroll
        for (int s = 0; s < S; ++s) acc[s] = (v4f){0.f, 0.f, 0.f, 0.f};
        // batches of NPF K blocks: all loads of a batch are issued back to back, then consumed in order; the other
        // wavefronts of the compute unit (up to 16) are at other points of their batches
        for (int kb = 0; kb < nkb; kb += NPF) {
#pragma unroll
            for (int p = 0; p < NPF; ++p)
                if (kb + p < nkb) fetch(p, kb + p);
#pragma unroll
            for (int p = 0; p < NPF; ++p) {
                if (kb + p < nkb) {                         // wavefront-uniform
                    const v8i af = join(alo[p], ahi[p]);
                    const float sc = sa[p] * sb[p];
#pragma unroll
                    for (int s = 0; s < S; ++s) {
                        const v8i wf = untangle(wlo[p][s], whi[p][s]);
                        const v4f z = {0.f, 0.f, 0.f, 0.f};
                        const v4f p4 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, z, 0, 0, 0, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[s][e] = __builtin_fmaf(p4[e], sc, acc[s][e]);
                    }
                }
            }
        }

        // add the wavefronts' partial sums in a fixed order, then store: lane (fr, fq) of strip s holds
        // c[row fr][n0 + 16 s + 4 fq .. +3]
        if (pass > 0) __syncthreads();
#pragma unroll
        for (int s = 0; s < S; ++s) red[(wave * S + s) * 64 + lane] = acc[s];
        __syncthreads();
        for (int slot_i = tid; slot_i < S * 64; slot_i += kWaves * kWave) {
            v4f v = red[slot_i];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                const v4f u = red[w * S * 64 + slot_i];
                v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
            }
            const int s = slot_i >> 6, l = slot_i & 63;
            const int m = l & 15, n = n0 + s * 16 + (l >> 4) * 4;
            if (m >= m_here) continue;
            const size_t idx = (size_t)(row0 + pass + m) * N + n;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e >= N) break;
                if (c_dtype == DSV3_F32)       ((float*)c)[idx + e] = v[e];
                else if (c_dtype == DSV3_BF16) ((uint16_t*)c)[idx + e] = cvt_out<DSV3_BF16>(v[e]);
                else                           ((uint16_t*)c)[idx + e] = cvt_out<DSV3_F16>(v[e]);
            }
        }
    }
}

}  // namespace gskinny

// Chosen by the caller for launches with few rows in all (every slot then has few rows); any table is computed
// correctly.
int launch_grouped_skinny(const void* a, const float* a_s, const int* a_rows, const void* b, const float* b_s, void* c,
                          int c_dtype, int64_t n, int64_t k, int64_t num_tiles, const int* tile_group,
                          const int* tile_row0, const int* tile_rows, int64_t b_stride, int64_t bs_stride,
                          int64_t groups_hint, hipStream_t stream) {
    using namespace gskinny;
    const int single_rows = 0;
    const int64_t strips = (n + 16 * S - 1) / (16 * S);
    if (strips > 0x7fffffff || num_tiles > 65535) return DSV3_ERR_BAD_SHAPE;
    if (strips == 0 || num_tiles == 0) return DSV3_OK;
    // wavefronts per workgroup (they split K), measured on the two GEMMs of the 256-expert layer: about 8 K blocks
    // per wavefront for a short K (2048: two wavefronts, 24 against 31 us with four at one token); for a long K
    // (7168) four wavefronts while the launch has few workgroups and eight once it has thousands of them
    // (one token: 46 against 50 us; eight tokens: 215 against 228 us).  `groups_hint` is the caller's estimate of
    // the live tile slots.
    const int64_t kb = k / 128;
    int waves = kb < 32 ? 2 : 4;
    if (kb >= 48 && strips * groups_hint >= 4096) waves = 8;
    static const int forced = getenv("DSV3_GS_WAVES") ? atoi(getenv("DSV3_GS_WAVES")) : 0;
    if (forced) waves = forced;
#define DSV3_GS(W)                                                                                                     \
    hipLaunchKernelGGL(fp8_gemm_grouped_skinny_kernel<W>, dim3((unsigned)strips, (unsigned)num_tiles), dim3(W * kWave), \
                       0, stream, (const uint8_t*)a, a_s, a_rows, (const uint8_t*)b, b_s, c, c_dtype, (int)n, (int)k,  \
                       tile_group, tile_row0, tile_rows, b_stride, bs_stride, single_rows)
    if (waves >= 16) DSV3_GS(16);
    else if (waves >= 8) DSV3_GS(8);
    else if (waves >= 4) DSV3_GS(4);
    else DSV3_GS(2);
#undef DSV3_GS
    return launch_status();
}

// The same kernel as ONE group without a tile table: a dense fp8_gemm with m <= 16 rows on a weight large enough
// that 32-row strips fill the chip.  No workspace and no second pass (the wavefronts of a workgroup split K).
bool skinny_single_supported(int64_t m, int64_t n, int64_t k) {
    return m >= 1 && m <= 16 && k >= 128 && k % 128 == 0 && n >= 1 && n * k < (1ll << 32) && m * k < (1ll << 32);
}

int launch_skinny_single(const void* a, const float* a_s, const void* b, const float* b_s, void* c, int c_dtype,
                         int64_t m, int64_t n, int64_t k, hipStream_t stream) {
    using namespace gskinny;
    const int64_t strips = (n + 16 * S - 1) / (16 * S), kb = k / 128;
    if (strips > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    // measured on 16384 -> 7168 (224 strips): 8 wavefronts 25.3 us, 4: 29.9, 16: 26.3
    const int waves = kb < 32 ? 2 : ((strips * 4 < 2048 && kb >= 64) ? 8 : 4);
    const int* none = nullptr;
    const int single_rows = (int)m;
#define DSV3_GS(W)                                                                                                     \
    hipLaunchKernelGGL(fp8_gemm_grouped_skinny_kernel<W>, dim3((unsigned)strips, 1u), dim3(W * kWave), 0, stream,      \
                       (const uint8_t*)a, a_s, none, (const uint8_t*)b, b_s, c, c_dtype, (int)n, (int)k, none, none,   \
                       none, (int64_t)0, (int64_t)0, single_rows)
    if (waves == 8) DSV3_GS(8);
    else if (waves == 4) DSV3_GS(4);
    else DSV3_GS(2);
#undef DSV3_GS
    return launch_status();
}

}  // namespace dsv3
