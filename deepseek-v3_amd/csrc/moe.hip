// Stream kernels around the grouped fp8_gemm of a mixture-of-experts layer
// (reference: inference/model.py:601-633 Expert, :669-693 MoE.forward).
//
//   swiglu_quant   g = silu(h1) * h3 rounded as the reference's bf16 tensor ops round it, then act_quant(g)
//                  (inference/model.py:633 feeding Linear -> inference/kernel.py:23-35) in one pass
//   moe_combine    y[t] = (sum over the token's experts, ascending expert index, of out * weight) + shared,
//                  every step rounded to bf16 exactly where model.py:689-693 rounds
//   group_tiles    per-group row counts -> the tile table the grouped GEMM reads (no host round trip)
//   moe_route      expert indices of every token -> per-expert counts, expert-sorted token list, and for every
//                  token its rows in that list in ascending expert order (what torch.where / bincount / the loop
//                  order of model.py:683-689 determine), in four small launches and without a sort
#include "common.hpp"

namespace dsv3 {
namespace {

constexpr int kThreads = 256;

// h: [rows, 2*inter] bf16 (h1 | h3 side by side), y: [rows, inter] e4m3, s: [rows, inter/128].
// A lane owns 8 consecutive output columns; the 16 lanes of a DPP row own one 128-wide scale block.
template <bool UE8M0>
__global__ __launch_bounds__(kThreads) void swiglu_quant_kernel(
        const v4u* __restrict__ h, v2u* __restrict__ y, float* __restrict__ s,
        int64_t n_chunks, int chunks_per_row) {
    const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const bool live = c < n_chunks;
    const int64_t cc = live ? c : 0;
    const int64_t row = cc / chunks_per_row;
    const int col = (int)(cc - row * chunks_per_row);
    const v4u a = __builtin_nontemporal_load(h + row * 2 * chunks_per_row + col);
    const v4u b = __builtin_nontemporal_load(h + row * 2 * chunks_per_row + chunks_per_row + col);
    // silu(h1) * h3 with the roundings of the reference's bf16 tensors (swiglu_bf16); the IEEE division unless every
    // |x| of the wavefront is below 64
    float x1[8], x3[8], g[8], big = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        x1[i] = (i & 1) ? bf16hi_to_f32(a[i >> 1]) : bf16lo_to_f32(a[i >> 1]);
        x3[i] = (i & 1) ? bf16hi_to_f32(b[i >> 1]) : bf16lo_to_f32(b[i >> 1]);
        big = fmaxf(big, fabsf(x1[i]));
    }
    if (__all(big < 64.f)) {            // (false for NaN as well)
#pragma unroll
        for (int i = 0; i < 8; ++i) g[i] = live ? swiglu_bf16<true>(x1[i], x3[i]) : 0.f;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) g[i] = live ? swiglu_bf16<false>(x1[i], x3[i]) : 0.f;
    }
    uint32_t abits = 0u;             // non-finite values reach the scale as in act_quant
#pragma unroll
    for (int i = 0; i < 8; ++i) abits = umax_u32(abits, abs_bits(g[i]));
    abits = dpp_umax<0xB1>(abits);   // quad_perm [1,0,3,2]
    abits = dpp_umax<0x4E>(abits);   // quad_perm [2,3,0,1]
    abits = dpp_umax<0x141>(abits);  // row_half_mirror
    abits = dpp_umax<0x140>(abits);  // row_mirror
    const float sc = block_scale(abits, UE8M0);
    // correctly rounded g / sc for bf16 g with |g| <= amax (same evaluation as act_quant)
    float q[8];
    if (block_is_finite(abits)) {
        const float r = 1.0f / sc;
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = block_quotient(g[i], sc, r, true);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = block_quotient(g[i], sc, 0.f, false);
    }
    if (live) {
        v2u o;
        o.x = pack_fp8x4(q[0], q[1], q[2], q[3]);
        o.y = pack_fp8x4(q[4], q[5], q[6], q[7]);
        __builtin_nontemporal_store(o, &y[c]);
        if ((c & 15) == 0) s[c >> 4] = sc;
    }
}

// One thread per 16-byte chunk of a token's output row (grid: tokens x chunk blocks).  rows[t, k] is the row of
// `out` holding the token's k-th expert output in ascending expert order, w[t, k] the matching routing weight
// (bf16).  The additions are a dependent chain of bf16 roundings, the loads are not: eight experts' chunks are
// fetched before they are added.
__global__ __launch_bounds__(kThreads) void moe_combine_kernel(
        const v4u* __restrict__ out, const int* __restrict__ rows, const uint16_t* __restrict__ w,
        const v4u* __restrict__ shared, v4u* __restrict__ y, int topk, int chunks_per_row) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * (int)blockDim.x + threadIdx.x;
    if (c >= chunks_per_row) return;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    v4u z = {0u, 0u, 0u, 0u};
    if (shared) z = shared[(int64_t)t * chunks_per_row + c];
    constexpr int U = 8;                      // expert rows fetched before they are added
    for (int k0 = 0; k0 < topk; k0 += U) {
        v4u v[U];
        float wk[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = min(k0 + u, topk - 1);
            wk[u] = bf16lo_to_f32(w[(int64_t)t * topk + k]);
            v[u] = __builtin_nontemporal_load(out + (int64_t)rows[(int64_t)t * topk + k] * chunks_per_row + c);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k0 + u < topk) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float x = (i & 1) ? bf16hi_to_f32(v[u][i >> 1]) : bf16lo_to_f32(v[u][i >> 1]);
                    acc[i] = round_bf16(acc[i] + round_bf16(x * wk[u]));       // y[idx] += expert_out * weight
                }
            }
        }
    }
    if (shared) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float x = (i & 1) ? bf16hi_to_f32(z[i >> 1]) : bf16lo_to_f32(z[i >> 1]);
            acc[i] = round_bf16(acc[i] + x);                                     // y + z
        }
    }
    v4u o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_bf16(acc[2 * i], acc[2 * i + 1]);
    y[(int64_t)t * chunks_per_row + c] = o;
}

// counts[g] rows per group, groups laid out back to back in c.  Tile slots are handed out group by group,
// ceil(count / tile_rows) each; slots past the last one are marked unused.  Called by every thread of ONE workgroup
// of kThreads threads; counts and offsets may live in LDS or in global memory.
__device__ __forceinline__ void tiles_from_counts(
        const int* counts, int groups, int tile_rows, int max_tiles,
        int* __restrict__ tile_group, int* __restrict__ tile_row0, int* __restrict__ tile_nrows,
        int* offsets) {                        // optional: first row of every group
    // Exclusive scans of (tiles, rows) over the groups, kThreads groups per batch: lane shuffles inside a
    // wavefront, the wavefronts' totals through LDS -- two barriers per batch.
    constexpr int kWaves = kThreads / kWave;
    __shared__ int wave_tiles[2][kWaves], wave_rows[2][kWaves];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int done_tiles = 0, done_rows = 0;
    for (int g0 = 0, batch = 0; g0 < groups; g0 += kThreads, ++batch) {
        const int g = g0 + threadIdx.x;
        const int cnt = g < groups ? counts[g] : 0;
        const int nt = (cnt + tile_rows - 1) / tile_rows;
        int st = nt, sr = cnt;                 // inclusive scans over the wavefront
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const int a = __shfl_up(st, d), b = __shfl_up(sr, d);
            if (lane >= d) { st += a; sr += b; }
        }
        int* wt = wave_tiles[batch & 1]; int* wr = wave_rows[batch & 1];      // (alternating: one barrier per batch)
        if (lane == kWave - 1) { wt[wave] = st; wr[wave] = sr; }
        __syncthreads();
        int t0 = done_tiles + st - nt, r0 = done_rows + sr - cnt, all_t = 0, all_r = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            if (w < wave) { t0 += wt[w]; r0 += wr[w]; }
            all_t += wt[w]; all_r += wr[w];
        }
        if (offsets && g < groups) offsets[g] = r0;
        for (int i = 0; i < nt; ++i) {
            if (t0 + i < max_tiles) {
                tile_group[t0 + i] = g;
                tile_row0[t0 + i] = r0 + i * tile_rows;
                tile_nrows[t0 + i] = min(tile_rows, cnt - i * tile_rows);
            }
        }
        done_tiles += all_t; done_rows += all_r;
    }
    for (int t = done_tiles + threadIdx.x; t < max_tiles; t += kThreads) {
        tile_group[t] = -1; tile_row0[t] = 0; tile_nrows[t] = 0;
    }
}

__global__ __launch_bounds__(kThreads) void group_tiles_kernel(
        const int* __restrict__ counts, int groups, int tile_rows, int max_tiles,
        int* __restrict__ tile_group, int* __restrict__ tile_row0, int* __restrict__ tile_nrows,
        int* __restrict__ offsets) {
    tiles_from_counts(counts, groups, tile_rows, max_tiles, tile_group, tile_row0, tile_nrows, offsets);
}

__global__ __launch_bounds__(kThreads) void fill_zero_kernel(int* __restrict__ p, int n) {
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (i < n) p[i] = 0;
}

// counts[e] += number of (token, slot) pairs routed to expert e; a workgroup first adds up its pairs in LDS
__global__ __launch_bounds__(kThreads) void route_count_kernel(
        const int64_t* __restrict__ indices, int64_t pairs, int experts, int* __restrict__ counts, int shared_rows) {
    extern __shared__ int bins[];
    if (shared_rows && blockIdx.x == 0 && threadIdx.x == 0) counts[experts] = shared_rows;   // nobody else adds to it
    for (int e = threadIdx.x; e < experts; e += kThreads) bins[e] = 0;
    __syncthreads();
    for (int64_t p = (int64_t)blockIdx.x * kThreads + threadIdx.x; p < pairs; p += (int64_t)gridDim.x * kThreads) {
        const int64_t e = indices[p];
        if (e >= 0 && e < experts) atomicAdd(&bins[e], 1);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += kThreads)
        if (bins[e]) atomicAdd(&counts[e], bins[e]);
}

// One thread per (token, slot) pair: the pair takes the next free row of its expert's group.  `rows` lists a
// token's pairs in ascending expert order -- the order in which the reference's loop adds them -- so a pair finds
// its place by counting the token's other entries that sort before it (smaller expert, or the same expert in an
// earlier slot: the order a stable sort gives).  The order of rows inside a group depends on the order in which
// threads arrive, which is harmless: a row of the grouped GEMM does not depend on its position, and `rows`
// records where each pair went.  With `shared_one` != 0 every token also takes row t of one more group (index
// `experts`, rows in token order) as its last entry, with that 16-bit pattern (1.0 in the weights' type) as its
// weight: the outputs then have topk + 1 columns.
__device__ __forceinline__ void scatter_pair(
        int64_t p, const int64_t* __restrict__ indices, const uint16_t* __restrict__ weights, int topk, int experts,
        const int* offsets, int* cursor, int* __restrict__ a_rows, int* __restrict__ rows,
        uint16_t* __restrict__ w_sorted, int shared_one) {
    const int t = (int)(p / topk), j0 = (int)(p - (int64_t)t * topk);
    const int cols = topk + (shared_one ? 1 : 0);
    const int64_t e = indices[p];
    int rank = 0;
    for (int j = 0; j < topk; ++j) {
        const int64_t o = indices[(int64_t)t * topk + j];
        rank += (o < e || (o == e && j < j0)) ? 1 : 0;
    }
    int pos = 0;
    if (e >= 0 && e < experts) {
        pos = offsets[e] + atomicAdd(&cursor[e], 1);
        a_rows[pos] = t;
    }
    rows[(int64_t)t * cols + rank] = pos;
    w_sorted[(int64_t)t * cols + rank] = weights[p];
    if (shared_one && j0 == 0) {
        const int spos = offsets[experts] + t;
        a_rows[spos] = t;
        rows[(int64_t)t * cols + topk] = spos;
        w_sorted[(int64_t)t * cols + topk] = (uint16_t)shared_one;
    }
}

// Many tokens: a workgroup first ranks its kThreads pairs per expert in LDS and then takes one range of rows per
// expert it holds with a single global atomic -- a popular expert otherwise serialises one atomic per row.
__global__ __launch_bounds__(kThreads) void route_scatter_pairs_kernel(
        const int64_t* __restrict__ indices, const uint16_t* __restrict__ weights, int64_t pairs, int topk, int experts,
        const int* __restrict__ offsets, int* __restrict__ cursor,
        int* __restrict__ a_rows, int* __restrict__ rows, uint16_t* __restrict__ w_sorted, int shared_one) {
    extern __shared__ int lds_i[];
    int* held = lds_i;                      // pairs of this workgroup per expert, then the first row of its range
    for (int e = threadIdx.x; e < experts; e += kThreads) held[e] = 0;
    __syncthreads();
    const int64_t p = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t e = p < pairs ? indices[p] : -1;
    const bool routed = e >= 0 && e < experts;
    const int local = routed ? atomicAdd(&held[e], 1) : 0;
    __syncthreads();
    for (int x = threadIdx.x; x < experts; x += kThreads)
        if (held[x]) held[x] = offsets[x] + atomicAdd(&cursor[x], held[x]);
    __syncthreads();
    if (p >= pairs) return;
    const int t = (int)(p / topk), j0 = (int)(p - (int64_t)t * topk);
    const int cols = topk + (shared_one ? 1 : 0);
    int rank = 0;
    for (int j = 0; j < topk; ++j) {
        const int64_t o = indices[(int64_t)t * topk + j];
        rank += (o < e || (o == e && j < j0)) ? 1 : 0;
    }
    int pos = 0;
    if (routed) {
        pos = held[e] + local;
        a_rows[pos] = t;
    }
    rows[(int64_t)t * cols + rank] = pos;
    w_sorted[(int64_t)t * cols + rank] = weights[p];
    if (shared_one && j0 == 0) {
        const int spos = offsets[experts] + t;
        a_rows[spos] = t;
        rows[(int64_t)t * cols + topk] = spos;
        w_sorted[(int64_t)t * cols + topk] = (uint16_t)shared_one;
    }
}

// The whole bookkeeping in one workgroup, for token counts up to kThreads (decode steps): counts, offsets and
// cursors stay in LDS; only the counts are also written out.
__global__ __launch_bounds__(kThreads) void route_small_kernel(
        const int64_t* __restrict__ indices, const uint16_t* __restrict__ weights, int tokens, int topk, int experts,
        int groups, int tile_rows, int max_tiles, int* __restrict__ counts_out, int* __restrict__ offsets_out,
        int* __restrict__ a_rows, int* __restrict__ rows, uint16_t* __restrict__ w_sorted,
        int* __restrict__ tile_group, int* __restrict__ tile_row0, int* __restrict__ tile_nrows, int shared_one) {
    extern __shared__ int lds_i[];
    int* bins = lds_i; int* offs = lds_i + groups; int* cur = lds_i + 2 * groups;
    for (int g = threadIdx.x; g < 3 * groups; g += kThreads) lds_i[g] = 0;
    __syncthreads();
    const int t = threadIdx.x;
    if (t < tokens) {
        for (int j = 0; j < topk; ++j) {
            const int64_t e = indices[(int64_t)t * topk + j];
            if (e >= 0 && e < experts) atomicAdd(&bins[e], 1);
        }
    }
    if (shared_one && t == 0) bins[experts] = tokens;
    __syncthreads();
    for (int g = threadIdx.x; g < groups; g += kThreads) counts_out[g] = bins[g];
    tiles_from_counts(bins, groups, tile_rows, max_tiles, tile_group, tile_row0, tile_nrows, offs);
    __syncthreads();
    for (int g = threadIdx.x; g < groups; g += kThreads) offsets_out[g] = offs[g];
    for (int p = threadIdx.x; p < tokens * topk; p += kThreads)
        scatter_pair(p, indices, weights, topk, experts, offs, cur, a_rows, rows, w_sorted, shared_one);
}

}  // namespace

int launch_moe_route(const int64_t* indices, const void* weights, int64_t tokens, int topk, int experts,
                     int shared_one, int max_tiles, int tile_rows, int* counts, int* offsets, int* cursor, int* a_rows,
                     int* rows, void* w_sorted, int* tile_group, int* tile_row0, int* tile_nrows, hipStream_t st) {
    const int64_t pairs = tokens * topk;
    const int groups = experts + (shared_one ? 1 : 0);
    if (tokens <= kThreads && groups <= 4096) {
        hipLaunchKernelGGL(route_small_kernel, dim3(1), dim3(kThreads), (size_t)3 * groups * sizeof(int), st,
                           indices, (const uint16_t*)weights, (int)tokens, topk, experts, groups, tile_rows, max_tiles,
                           counts, offsets, a_rows, rows, (uint16_t*)w_sorted, tile_group, tile_row0, tile_nrows, shared_one);
        return launch_status();
    }
    // counts | offsets | cursor are consecutive thirds of one scratch array; clear it with a kernel (a memset node
    // recorded into a captured graph has given wrong results on replays)
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((3 * groups + kThreads - 1) / kThreads)), dim3(kThreads), 0, st, counts, 3 * groups);
    const unsigned cgrid = (unsigned)((pairs + kThreads * 8 - 1) / (kThreads * 8) > 1024 ? 1024 : (pairs + kThreads * 8 - 1) / (kThreads * 8));
    hipLaunchKernelGGL(route_count_kernel, dim3(cgrid ? cgrid : 1), dim3(kThreads), (size_t)experts * sizeof(int), st,
                       indices, pairs, experts, counts, shared_one ? (int)tokens : 0);
    hipLaunchKernelGGL(group_tiles_kernel, dim3(1), dim3(kThreads), 0, st,
                       (const int*)counts, groups, tile_rows, max_tiles, tile_group, tile_row0, tile_nrows, offsets);
    hipLaunchKernelGGL(route_scatter_pairs_kernel, dim3((unsigned)((pairs + kThreads - 1) / kThreads)), dim3(kThreads),
                       (size_t)experts * sizeof(int), st,
                       indices, (const uint16_t*)weights, pairs, topk, experts, (const int*)offsets, cursor,
                       a_rows, rows, (uint16_t*)w_sorted, shared_one);
    return launch_status();
}

int launch_swiglu_quant(const void* h, void* y, float* s, int64_t rows, int64_t inter, int scale_fmt, hipStream_t st) {
    const int64_t n_chunks = rows * inter / 8;
    const int64_t grid = (n_chunks + kThreads - 1) / kThreads;
    if (grid > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (scale_fmt == DSV3_SCALE_FMT_UE8M0)
        hipLaunchKernelGGL(swiglu_quant_kernel<true>, dim3((unsigned)grid), dim3(kThreads), 0, st,
                           (const v4u*)h, (v2u*)y, s, n_chunks, (int)(inter / 8));
    else
        hipLaunchKernelGGL(swiglu_quant_kernel<false>, dim3((unsigned)grid), dim3(kThreads), 0, st,
                           (const v4u*)h, (v2u*)y, s, n_chunks, (int)(inter / 8));
    return launch_status();
}

int launch_moe_combine(const void* out, const int* rows, const void* w, const void* shared, void* y,
                       int64_t tokens, int topk, int64_t dim, hipStream_t st) {
    // 128 threads where that leaves no partly filled workgroup (7168 columns = 896 chunks = 7 x 128)
    const int64_t chunks = dim / 8;
    const int threads = (chunks % kThreads != 0 && chunks % 128 == 0) ? 128 : kThreads;
    const unsigned chunk_blocks = (unsigned)((chunks + threads - 1) / threads);
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)tokens, chunk_blocks), dim3(threads), 0, st,
                       (const v4u*)out, rows, (const uint16_t*)w, (const v4u*)shared, (v4u*)y, topk, (int)(dim / 8));
    return launch_status();
}

int launch_group_tiles(const int* counts, int groups, int tile_rows, int max_tiles,
                       int* tile_group, int* tile_row0, int* tile_nrows, hipStream_t st) {
    hipLaunchKernelGGL(group_tiles_kernel, dim3(1), dim3(kThreads), 0, st,
                       counts, groups, tile_rows, max_tiles, tile_group, tile_row0, tile_nrows, (int*)nullptr);
    return launch_status();
}

}  // namespace dsv3
