// The two per-head products of the absorbed MLA attention with the block-scaled fp8 weight wkv_b, without
// materialising weight_dequant(wkv_b) (reference: inference/model.py:481-483 and :495).
//
//   wkv_b : fp8 [heads * (nope + v), C], scales fp32 [ceil(rows/128), C/128]; head h owns rows h*(nope+v) ...
//   W     : bf16( f32(wkv_b) * scale )        -- exactly what weight_dequant would have written (kernel.py:83-86)
//   side Q: y[m, h, c] = sum_d x[m, h, d] * W[h*(nope+v) + d,        c]     d < nope   ("bshd,hdc->bshc")
//   side V: y[m, h, d] = sum_c x[m, h, c] * W[h*(nope+v) + nope + d, c]     d < v      ("bshc,hdc->bshd")
//
// Both are weight-stationary: a wavefront dequantises one slab of one head's weight ONCE into MFMA operand
// registers (128 VGPRs of bf16: 128 x 128 for side Q, 32 x 512 for side V), then streams 16-token sub-tiles
// past it with v_mfma_f32_16x16x32_bf16.  Operand roles are picked per side so that a lane ends up with
// consecutive output features of a token and writes them with 16-byte stores.  Which output feature sits in
// which MFMA row, and which K index sits in which operand slot, is free as long as both operands agree; the maps
// below are chosen so that every global access of a lane is one aligned 8- or 16-byte piece:
//
//   side Q  (K = d runs over weight ROWS, features c are contiguous in memory)
//     wave slab: 128 features c0 .. c0+127, 8 MFMA sub-tiles t; MFMA row i of sub-tile t is feature c0 + 8*i + t.
//     lane (i = lane%16, g = lane/16) reads, for each of its 8 K rows of a 32-row step, the 8 bytes
//     [c0 + 8*i, +8) -> byte t belongs to sub-tile t.  Side Q issues the activation as the A operand instead, so
//     the lane owns features c0 + 8*i + [0, 8) of the four tokens 4*g .. 4*g+3 and a group of 16 lanes writes 256
//     contiguous bytes of one token.
//   side V  (K = c is contiguous in memory, features d are weight rows)
//     wave slab: 32 features d0 .. d0+31, 2 sub-tiles; MFMA row i of sub-tile t is feature d0 + 8*(i/4) + 4*t + i%4.
//     Within a 128-wide K block lane group g takes the 32 consecutive K values [32*g, +32) (four MFMA steps), so
//     a lane reads 32 contiguous weight bytes and 64 contiguous activation bytes per K block, all inside one scale
//     block.  It owns output features d0 + 8*g + [0, 8) of token i.
//
// HBM traffic: the weight slab once per workgroup (8.4 MB per side for the 671B shape), the activations once
// (the four wavefronts of a workgroup share their reads through the L1), the output once.
#include "common.hpp"

namespace dsv3 {
namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

__device__ __forceinline__ v4f mfma_bf16(v4u a, v4u b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
}

struct AbsorbArgs {
    const uint16_t* x;      // bf16 activations
    int64_t x_ts, x_hs;     // token / head stride of x in elements
    const uint8_t* w;       // fp8 wkv_b
    const float* ws;        // its block scales
    int64_t w_cols;         // C
    int ws_cols;            // C / 128
    uint16_t* y;            // bf16 [tokens, heads, n_out]
    int64_t tokens;
    int heads, head_rows, nope, n_out;
    int slabs;              // feature slabs per head (side Q: C/128, side V: v/32)
    int subtiles;           // ceil(tokens / 16)
};

// 8 fp8 bytes -> 8 binary32
__device__ __forceinline__ void cvt8(v2u p, float (&f)[8]) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        v2f lo = fp8x2_lo_to_f32(p[q]), hi = fp8x2_hi_to_f32(p[q]);
        f[4 * q] = lo.x; f[4 * q + 1] = lo.y; f[4 * q + 2] = hi.x; f[4 * q + 3] = hi.y;
    }
}

// side Q; KS = nope / 32 MFMA K steps; NT: write the output with non-temporal stores (outputs far larger than the
// last-level cache, which the next kernel could not find there anyway)
template <int KS, bool NT>
__global__ __launch_bounds__(256) void absorb_q_kernel(AbsorbArgs p) {
    const int lane = threadIdx.x & 63;
    const int slab = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (slab >= p.slabs) return;
    const int h = blockIdx.y, i = lane & 15, g = lane >> 4;
    const int c0 = slab * 128;
    const int64_t row0 = (int64_t)h * p.head_rows;

    v4u A[KS][8];
    {
        v2u raw[KS][8];
        float sc[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int64_t r = row0 + s * 32 + g * 8;       // 8 rows r .. r+7 lie in one scale block
            sc[s] = p.ws[(r >> 7) * p.ws_cols + slab];
#pragma unroll
            for (int e = 0; e < 8; ++e) raw[s][e] = *(const v2u*)(p.w + (r + e) * p.w_cols + c0 + i * 8);
        }
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                float f0[8], f1[8];
                cvt8(raw[s][2 * e2], f0);
                cvt8(raw[s][2 * e2 + 1], f1);
#pragma unroll
                for (int t = 0; t < 8; ++t) A[s][t][e2] = pack_bf16(f0[t] * sc[s], f1[t] * sc[s]);
            }
    }

    // The token loop has no branches besides its back edge: rows past the end are clamped to the last token (they
    // load, compute and store that token's values again) and the prefetch past the last sub-tile repeats it, so
    // the compiler can count the stores that follow each prefetch instead of draining them (s_waitcnt vmcnt(4)).
    const uint16_t* xh = p.x + (int64_t)h * p.x_hs + g * 8;
    const int64_t last = p.tokens - 1;
    auto load_b = [&](int ms, v4u (&b)[KS]) {
        ms = ms < p.subtiles ? ms : p.subtiles - 1;
        int64_t tok = (int64_t)ms * 16 + i;
        tok = tok < last ? tok : last;
        const uint16_t* src = xh + tok * p.x_ts;
#pragma unroll
        for (int s = 0; s < KS; ++s) b[s] = *(const v4u*)(src + s * 32);
    };

    v4u bn[KS];
    load_b(blockIdx.z, bn);
    for (int ms = blockIdx.z; ms < p.subtiles; ms += gridDim.z) {
        v4u b[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) b[s] = bn[s];
        load_b(ms + gridDim.z, bn);
        // activations are the MFMA A operand here: the lane gets feature column i of sub-tile t (feature
        // c0 + 8*i + t) for the four tokens 4*g + j, i.e. 8 consecutive features per token, and the 16 lanes of a
        // group write one token's 128 features of this slab as 256 contiguous bytes
        v4f acc[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int t = 0; t < 8; ++t) acc[t] = mfma_bf16(b[s], A[s][t], acc[t]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int64_t tok = (int64_t)ms * 16 + g * 4 + j;
            tok = tok < last ? tok : last;
            v4u o;
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = pack_bf16(acc[2 * q][j], acc[2 * q + 1][j]);
            v4u* dst = (v4u*)(p.y + (tok * p.heads + h) * p.n_out + c0 + i * 8);
            if (NT) __builtin_nontemporal_store(o, dst);
            else *dst = o;
        }
    }
}

// side V; KB = C / 128 scale blocks along K
template <int KB>
__global__ __launch_bounds__(256) void absorb_v_kernel(AbsorbArgs p) {
    const int lane = threadIdx.x & 63;
    const int slab = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (slab >= p.slabs) return;
    const int h = blockIdx.y, i = lane & 15, g = lane >> 4;
    const int d0 = slab * 32;
    const int64_t row0 = (int64_t)h * p.head_rows + p.nope + d0;

    v4u A[2][KB][4];
    {
        v4u raw[2][KB][2];
        float sc[2][KB];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int64_t r = row0 + (i >> 2) * 8 + t * 4 + (i & 3);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                sc[t][kb] = p.ws[(r >> 7) * p.ws_cols + kb];
                const v4u* src = (const v4u*)(p.w + r * p.w_cols + kb * 128 + g * 32);
                raw[t][kb][0] = src[0];
                raw[t][kb][1] = src[1];
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    // K values 8*s .. 8*s+7 of the lane's 32: dwords 2*s and 2*s+1 of the 32 bytes
                    float f[8];
                    cvt8(v2u{raw[t][kb][s >> 1][2 * (s & 1)], raw[t][kb][s >> 1][2 * (s & 1) + 1]}, f);
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        A[t][kb][s][q] = pack_bf16(f[2 * q] * sc[t][kb], f[2 * q + 1] * sc[t][kb]);
                }
    }

    // The token loop has no branches besides its back edge (see side Q).  A sub-tile is consumed in NS steps of KH
    // K blocks; while one step's activations feed the MFMAs the next step's are in flight.
    constexpr int NS = KB >= 2 ? 2 : 1, KH = KB / NS;
    const uint16_t* xh = p.x + (int64_t)h * p.x_hs + g * 32;
    const int64_t last = p.tokens - 1;
    auto load_b = [&](int ms, int step, v4u (&b)[KH][4]) {
        ms = ms < p.subtiles ? ms : p.subtiles - 1;
        int64_t tok = (int64_t)ms * 16 + i;
        tok = tok < last ? tok : last;
        const uint16_t* src = xh + tok * p.x_ts + step * (KH * 128);
#pragma unroll
        for (int kb = 0; kb < KH; ++kb)
#pragma unroll
            for (int s = 0; s < 4; ++s) b[kb][s] = *(const v4u*)(src + kb * 128 + s * 8);
    };

    v4u bn[KH][4];
    load_b(blockIdx.z, 0, bn);
    for (int ms = blockIdx.z; ms < p.subtiles; ms += gridDim.z) {
        // two accumulators per sub-tile (even / odd K steps) keep four independent MFMA chains in flight
        v4f acc[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[t][0] = acc[t][1] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int step = 0; step < NS; ++step) {
            v4u b[KH][4];
#pragma unroll
            for (int kb = 0; kb < KH; ++kb)
#pragma unroll
                for (int s = 0; s < 4; ++s) b[kb][s] = bn[kb][s];
            if (step + 1 < NS) load_b(ms, step + 1, bn);
            else load_b(ms + gridDim.z, 0, bn);
#pragma unroll
            for (int kb = 0; kb < KH; ++kb)
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                        acc[t][s & 1] = mfma_bf16(A[t][step * KH + kb][s], b[kb][s], acc[t][s & 1]);
        }
        int64_t tok = (int64_t)ms * 16 + i;
        tok = tok < last ? tok : last;            // clamped rows rewrite the last token's values
        v4u o;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const v4f r = acc[t][0] + acc[t][1];
            o[2 * t] = pack_bf16(r[0], r[1]);
            o[2 * t + 1] = pack_bf16(r[2], r[3]);
        }
        *(v4u*)(p.y + (tok * p.heads + h) * p.n_out + d0 + g * 8) = o;
    }
}


// side V for more than 64 tokens, C == 512, v % 128 == 0: same weight slabs and MFMA maps as absorb_v_kernel, but the
// activations reach the MFMAs through LDS.  Read straight from global memory, a B fragment is 64 pieces of 16
// bytes from 16 different token rows per load instruction, and each of the four wavefronts of a workgroup
// fetches the whole 1 KiB row of a token again; that pattern, not HBM, bounds absorb_v_kernel once the weights
// are amortised.  Here a wavefront's load instruction moves one whole token row (64 lanes x 16 bytes, contiguous)
// with global_load_lds_dwordx4, each row is fetched once per workgroup, and the fragments come from LDS.
//
// LDS: S stages of 16 rows x 1 KiB.  The 16-byte chunk c of row r is stored at chunk position c ^ (r & 15)
// (the permutation is applied to the global address a lane loads from, since the LDS side of the load is fixed
// to lane order), which spreads the 16 rows of a ds_read_b128 over all banks.
//
// Pipeline per workgroup iteration: wait for the oldest stage's loads (own vmcnt; loads and stores retire in
// issue order, so the later ones are simply counted), barrier, refill the stage everybody finished reading one
// iteration ago, read fragments, multiply, store.
constexpr int kStagedRows = 16, kStagedRowBytes = 1024, kStagedStage = kStagedRows * kStagedRowBytes;
typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int S>
__global__ __launch_bounds__(256) void absorb_v_staged_kernel(AbsorbArgs p) {
    constexpr int KB = 4;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slab = blockIdx.x * 4 + wave;                 // slabs is a multiple of 4 here
    const int h = blockIdx.y, i = lane & 15, g = lane >> 4;
    const int d0 = slab * 32;
    const int64_t row0 = (int64_t)h * p.head_rows + p.nope + d0;

    v4u A[2][KB][4];
    {
        v4u raw[2][KB][2];
        float sc[2][KB];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int64_t r = row0 + (i >> 2) * 8 + t * 4 + (i & 3);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                sc[t][kb] = p.ws[(r >> 7) * p.ws_cols + kb];
                const v4u* src = (const v4u*)(p.w + r * p.w_cols + kb * 128 + g * 32);
                raw[t][kb][0] = src[0];
                raw[t][kb][1] = src[1];
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    float f[8];
                    cvt8(v2u{raw[t][kb][s >> 1][2 * (s & 1)], raw[t][kb][s >> 1][2 * (s & 1) + 1]}, f);
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        A[t][kb][s][q] = pack_bf16(f[2 * q] * sc[t][kb], f[2 * q + 1] * sc[t][kb]);
                }
    }
    // the weight loads above must not be counted among the loads the pipeline waits for
    __builtin_amdgcn_s_waitcnt(0x0f70);

    const int64_t last = p.tokens - 1;
    const int gz = gridDim.z;
    const uint16_t* xh = p.x + (int64_t)h * p.x_hs;
    // wavefront `wave` moves rows wave, wave+4, wave+8, wave+12 of a tile (one instruction each)
    auto issue_tile = [&](int ms, int stage) {
        ms = ms < p.subtiles ? ms : p.subtiles - 1;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const int r = n * 4 + wave;
            int64_t tok = (int64_t)ms * 16 + r;
            tok = tok < last ? tok : last;
            const uint16_t* src = xh + tok * p.x_ts + ((lane ^ r) << 3);      // r < 16: permutes the low 4 chunk bits
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + stage * kStagedStage + r * kStagedRowBytes),
                                             16, 0, 0);
        }
    };
    // fragment (kb, s) of the lane: row i, chunk kb*16 + g*4 + s
    const uint8_t* frag = lds + i * kStagedRowBytes;
    int frag_off[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) frag_off[s] = (((g * 4 + s) ^ i) << 4);

    int ms = blockIdx.z;
#pragma unroll
    for (int t = 0; t < S - 1; ++t) issue_tile(ms + t * gz, t);
    int stage = 0;
    for (int it = 0; ms < p.subtiles; ms += gz, ++it) {
        // outstanding after the loads of this tile: the loads of the S-2 tiles behind it, and (once the
        // pipeline runs) one store per iteration since they were issued
        if (it < S - 1) __builtin_amdgcn_s_waitcnt(0x0f70 | (4 * (S - 2)));
        else            __builtin_amdgcn_s_waitcnt(0x0f70 | (4 * (S - 2) + (S - 1)));
        wg_barrier();
        issue_tile(ms + (S - 1) * gz, stage == 0 ? S - 1 : stage - 1);
        const uint8_t* st = frag + stage * kStagedStage;
        v4f acc[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[t][0] = acc[t][1] = v4f{0.f, 0.f, 0.f, 0.f};
        v4u b[2][4];                                  // K block kb+1 is read while kb feeds the MFMAs
#pragma unroll
        for (int s = 0; s < 4; ++s) b[0][s] = *(const v4u*)(st + frag_off[s]);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            if (kb + 1 < KB) {
#pragma unroll
                for (int s = 0; s < 4; ++s) b[(kb + 1) & 1][s] = *(const v4u*)(st + (kb + 1) * 256 + frag_off[s]);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t][s & 1] = mfma_bf16(A[t][kb][s], b[kb & 1][s], acc[t][s & 1]);
        }
        // keep the order written above (the scheduler otherwise sinks every read next to its use and waits for
        // each pair): 4 reads ahead, then per K block the next 4 reads followed by its 8 MFMAs
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            if (kb + 1 < KB) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        }
        int64_t tok = (int64_t)ms * 16 + i;
        tok = tok < last ? tok : last;
        v4u o;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const v4f r = acc[t][0] + acc[t][1];
            o[2 * t] = pack_bf16(r[0], r[1]);
            o[2 * t + 1] = pack_bf16(r[2], r[3]);
        }
        *(v4u*)(p.y + (tok * p.heads + h) * p.n_out + d0 + g * 8) = o;
        stage = stage + 1 == S ? 0 : stage + 1;
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);     // the clamped refills of the last iterations still write LDS
}


// Up to 256 tokens the conversion of the weight slab is the longest step of a wavefront that does it alone (a
// 128 x 128 slab is 256 values per lane before the first MFMA can start).  The kernels below give a slab to a
// workgroup of four wavefronts: each converts a quarter of it and leaves its MFMA operand fragments in LDS (one
// 16-byte piece per lane and fragment, lanes in order: no bank conflicts either way), and after one barrier every
// wavefront reads the whole slab's fragments back and takes every fourth 16-token sub-tile.  An output element is
// still formed by one wavefront over the whole K range in the same order, so the results are those of the kernels
// above bit for bit.
template <int KS, int PF>
__global__ __launch_bounds__(256) void absorb_q_shared_kernel(AbsorbArgs p) {
    __shared__ v4u frag[KS * 8 * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slab = blockIdx.y, h = blockIdx.x, i = lane & 15, g = lane >> 4;
    const int c0 = slab * 128;
    const int64_t row0 = (int64_t)h * p.head_rows;
    const int stride = gridDim.z * 4;
    const int ms0 = blockIdx.z * 4 + wave;

    const uint16_t* xh = p.x + (int64_t)h * p.x_hs + g * 8;
    const int64_t last = p.tokens - 1;
    auto load_b = [&](int ms, v4u (&b)[KS]) {
        ms = ms < p.subtiles ? ms : p.subtiles - 1;
        int64_t tok = (int64_t)ms * 16 + i;
        tok = tok < last ? tok : last;
        const uint16_t* src = xh + tok * p.x_ts;
#pragma unroll
        for (int s = 0; s < KS; ++s) b[s] = *(const v4u*)(src + s * 32);
    };
    v4u ring[PF][KS];                                      // PF sub-tiles' activations in flight, the first during the conversion
#pragma unroll
    for (int j = 0; j < PF; ++j) load_b(ms0 + j * stride, ring[j]);

    for (int s = wave; s < KS; s += 4) {
        const int64_t r = row0 + s * 32 + g * 8;           // 8 rows r .. r+7 lie in one scale block
        const float sc = p.ws[(r >> 7) * p.ws_cols + slab];
        v2u raw[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) raw[e] = *(const v2u*)(p.w + (r + e) * p.w_cols + c0 + i * 8);
        v4u a[8];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            float f0[8], f1[8];
            cvt8(raw[2 * e2], f0);
            cvt8(raw[2 * e2 + 1], f1);
#pragma unroll
            for (int t = 0; t < 8; ++t) a[t][e2] = pack_bf16(f0[t] * sc, f1[t] * sc);
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) frag[(s * 8 + t) * 64 + lane] = a[t];
    }
    __syncthreads();
    if (ms0 >= p.subtiles) return;
    v4u A[KS][8];
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int t = 0; t < 8; ++t) A[s][t] = frag[(s * 8 + t) * 64 + lane];

    for (int base = ms0; base < p.subtiles; base += PF * stride)
#pragma unroll
    for (int j = 0; j < PF; ++j) {
        const int ms = base + j * stride;
        if (ms >= p.subtiles) break;
        v4u b[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) b[s] = ring[j][s];
        load_b(ms + PF * stride, ring[j]);
        v4f acc[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int t = 0; t < 8; ++t) acc[t] = mfma_bf16(b[s], A[s][t], acc[t]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int64_t tok = (int64_t)ms * 16 + g * 4 + j;
            tok = tok < last ? tok : last;
            v4u o;
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = pack_bf16(acc[2 * q][j], acc[2 * q + 1][j]);
            *(v4u*)(p.y + (tok * p.heads + h) * p.n_out + c0 + i * 8) = o;
        }
    }
}

// Side V for up to 256 tokens, C == 512 and v == 128: the K range, not the features, is split over the wavefronts.
// A wavefront that owns a feature slab needs every byte of a token's 1 KiB activation row, so the four slabs of a
// head read each row four times (through the L1 at best, through the fabric when they sit on different XCDs), in
// scattered 16-byte pieces; with few tokens that, and a 16 KiB slab to convert per wavefront, is the whole time.
// Here a workgroup of eight wavefronts owns a head: wavefront (kb, dh) holds K block kb (128 values) of feature
// half dh (64 features) -- an 8 KiB slab, 64 registers of MFMA operands, half the conversion -- and reads only its
// quarter of each activation row.  The four K partial sums of an output meet in LDS: every wavefront leaves its four
// 16 x 16 partial tiles there and, after a barrier, adds up (in K order, whichever wavefront does it) the tile whose
// number equals its kb; two buffers alternate, so no barrier is needed behind the additions.  Feature map: MFMA row i of sub-tile t is feature
// dh*64 + 16*(i/4) + 4*t + i%4, so the lane (token i%16, group g) that reduces tile t ends with the four consecutive
// features dh*64 + 16*g + 4*t + [0, 4).  blockIdx.x is the head: the workgroups of a head (gridDim.z token groups)
// have the same index mod 8 and so share one XCD's L2 for the weight.
// The activations reach the MFMAs through LDS: read straight from global memory, a wavefront's fragment load is 64 pieces
// of 16 bytes at 64-byte stride in 16 rows; here the eight wavefronts copy a sub-tile's 16 rows whole (two 1 KiB rows
// each, global_load_lds_dwordx4, chunks xor-ed with the row as in absorb_v_staged_kernel), one sub-tile ahead, and read
// their fragments from LDS (64 tokens: 7.3 -> 6.95 us).  Two fence-free barriers per sub-tile: the copies have landed /
// the partial sums are written.
__global__ __launch_bounds__(512) void absorb_v_ksplit_kernel(AbsorbArgs p) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    v4f (*part)[8][4][64] = (v4f (*)[8][4][64])(lds + 2 * kStagedStage);       // [2][8][4][64]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kb = wave & 3, dh = wave >> 2;
    const int h = blockIdx.x, i = lane & 15, g = lane >> 4;
    const int64_t row0 = (int64_t)h * p.head_rows + p.nope + dh * 64;
    const int stride = gridDim.z;
    const int64_t last = p.tokens - 1;
    const uint16_t* xh = p.x + (int64_t)h * p.x_hs;
    auto issue_tile = [&](int ms, int stage) {                 // rows 2*wave and 2*wave + 1 of the sub-tile
        ms = ms < p.subtiles ? ms : p.subtiles - 1;
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const int r = wave * 2 + n;
            int64_t tok = (int64_t)ms * 16 + r;
            tok = tok < last ? tok : last;
            const uint16_t* src = xh + tok * p.x_ts + ((lane ^ r) << 3);
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + stage * kStagedStage + r * kStagedRowBytes), 16, 0, 0);
        }
    };
    issue_tile(blockIdx.z, 0);

    v4u A[4][4];
    {
        v4u raw[4][2];
        float sc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int64_t r = row0 + (i >> 2) * 16 + t * 4 + (i & 3);
            sc[t] = p.ws[(r >> 7) * p.ws_cols + kb];
            const v4u* src = (const v4u*)(p.w + r * p.w_cols + kb * 128 + g * 32);
            raw[t][0] = src[0];
            raw[t][1] = src[1];
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                float f[8];
                cvt8(v2u{raw[t][s >> 1][2 * (s & 1)], raw[t][s >> 1][2 * (s & 1) + 1]}, f);
#pragma unroll
                for (int q = 0; q < 4; ++q) A[t][s][q] = pack_bf16(f[2 * q] * sc[t], f[2 * q + 1] * sc[t]);
            }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);          // (weights and the first sub-tile's copies: nothing of them is counted below)

    // fragment s of the lane: row i, chunk kb*16 + g*4 + s, stored at chunk position (low four bits) ^ i
    int frag_off[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) frag_off[s] = i * kStagedRowBytes + ((kb * 16 + ((g * 4 + s) ^ i)) << 4);

    int it = 0;
    for (int ms = blockIdx.z; ms < p.subtiles; ms += stride, ++it) {
        const int st = it & 1;
        issue_tile(ms + stride, st ^ 1);          // the other stage was read before the last barrier of the iteration before
        // outstanding after this sub-tile's copies: the two just issued (the store of the iteration before is older)
        if (it > 0) __builtin_amdgcn_s_waitcnt(0x0f70 | 2);
        wg_barrier();
        v4u b[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) b[s] = *(const v4u*)(lds + st * kStagedStage + frag_off[s]);
        v4f acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[t] = mfma_bf16(A[t][s], b[s], acc[t]);
#pragma unroll
        for (int t = 0; t < 4; ++t) part[st][wave][t][lane] = acc[t];
        wg_barrier();
        v4f r = part[st][dh * 4 + 0][kb][lane];
#pragma unroll
        for (int w = 1; w < 4; ++w) r += part[st][dh * 4 + w][kb][lane];
        int64_t tok = (int64_t)ms * 16 + i;
        tok = tok < last ? tok : last;
        *(v2u*)(p.y + (tok * p.heads + h) * p.n_out + dh * 64 + g * 16 + kb * 4) = v2u{ pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]) };
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);          // the clamped copies of the last iteration still write LDS
}

}  // namespace

bool wkv_b_absorb_supported(int side, int nope, int v, int64_t kv_rank) {
    if (kv_rank <= 0 || kv_rank % 128 != 0 || nope % 32 != 0 || v % 32 != 0 || nope <= 0 || v <= 0) return false;
    if (side == DSV3_ABSORB_Q) return nope == 64 || nope == 128;
    return kv_rank == 128 || kv_rank == 256 || kv_rank == 512;
}

int launch_wkv_b_absorb(const void* x, int64_t x_ts, int64_t x_hs, const void* w, const float* ws, void* y, int side,
                        int64_t tokens, int heads, int nope, int v, int64_t kv_rank, hipStream_t st) {
    AbsorbArgs p;
    p.x = (const uint16_t*)x; p.x_ts = x_ts; p.x_hs = x_hs;
    p.w = (const uint8_t*)w; p.ws = ws; p.w_cols = kv_rank; p.ws_cols = (int)(kv_rank / 128);
    p.y = (uint16_t*)y; p.tokens = tokens; p.heads = heads; p.head_rows = nope + v; p.nope = nope;
    p.subtiles = (int)((tokens + 15) / 16);
    const bool q = side == DSV3_ABSORB_Q;
    p.n_out = q ? (int)kv_rank : v;
    p.slabs = q ? (int)(kv_rank / 128) : v / 32;
    if (!q && kv_rank == 512 && v == 128 && p.subtiles >= 3 && p.subtiles <= 8) {
        // 33 .. 128 tokens of side V: a head per workgroup, K split over its wavefronts; one workgroup per CU
        int gz = 256 / (heads > 0 ? heads : 1);
        gz = gz < 1 ? 1 : gz;
        gz = gz > p.subtiles ? p.subtiles : gz;
        constexpr int bytes = 2 * kStagedStage + 2 * 8 * 4 * 64 * 16;       // two activation stages + two buffers of partial sums
        static LdsGrant ks_grant;
        if (!ks_grant.ensure((const void*)absorb_v_ksplit_kernel, bytes)) return DSV3_ERR_LAUNCH;
        hipLaunchKernelGGL(absorb_v_ksplit_kernel, dim3(heads, 1, gz), dim3(512), bytes, st, p);
        return launch_status();
    }
    if (q && p.subtiles <= 16) {
        // up to 256 tokens of side Q: a slab per workgroup, its sub-tiles dealt over (gridDim.z, wavefront); the
        // head is blockIdx.x, so that the workgroups of a head share one XCD's L2
        int gz = (p.subtiles + 3) / 4;
        const int cap = 512 / (p.slabs * heads > 0 ? p.slabs * heads : 1);
        gz = gz > cap ? cap : gz;
        gz = gz < 1 ? 1 : gz;
        const dim3 grid(heads, p.slabs, gz), block(256);
        const bool one = (p.subtiles + 4 * gz - 1) / (4 * gz) <= 1;      // sub-tiles per wavefront
        if (nope == 128 && one) hipLaunchKernelGGL((absorb_q_shared_kernel<4, 1>), grid, block, 0, st, p);
        else if (nope == 128) hipLaunchKernelGGL((absorb_q_shared_kernel<4, 2>), grid, block, 0, st, p);
        else if (one) hipLaunchKernelGGL((absorb_q_shared_kernel<2, 1>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((absorb_q_shared_kernel<2, 2>), grid, block, 0, st, p);
        return launch_status();
    }
    // few tokens: one wavefront per workgroup spreads the weight reads over every CU; many tokens: the wavefronts
    // of a workgroup take different slabs of the same head and share the activation reads
    const int waves = p.subtiles > 4 ? 4 : 1;
    const int gx = (p.slabs + waves - 1) / waves;
    // token sub-tiles are dealt over gridDim.z so that about two workgroups per CU are resident
    int gz = 512 / (gx * heads > 0 ? gx * heads : 1);
    gz = gz < 1 ? 1 : gz;
    gz = gz > p.subtiles ? p.subtiles : gz;
    gz = gz > 65535 ? 65535 : gz;
    const dim3 grid(gx, heads, gz), block(64 * waves);
    if (!q && kv_rank == 512 && v % 128 == 0 && waves == 4) {
        constexpr int S = 4;
        static LdsGrant grant;                   // 64 KiB of dynamic LDS needs the opt-in once per device
        if (!grant.ensure((const void*)absorb_v_staged_kernel<S>, S * kStagedStage)) return DSV3_ERR_LAUNCH;
        hipLaunchKernelGGL(absorb_v_staged_kernel<S>, grid, block, S * kStagedStage, st, p);
        return launch_status();
    }
    if (q) {
        const bool nt = tokens * heads * kv_rank * 2 > (int64_t)256 << 20;
        if (nope == 128 && nt) hipLaunchKernelGGL((absorb_q_kernel<4, true>), grid, block, 0, st, p);
        else if (nope == 128) hipLaunchKernelGGL((absorb_q_kernel<4, false>), grid, block, 0, st, p);
        else if (nt) hipLaunchKernelGGL((absorb_q_kernel<2, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((absorb_q_kernel<2, false>), grid, block, 0, st, p);
    } else {
        if (kv_rank == 512) hipLaunchKernelGGL(absorb_v_kernel<4>, grid, block, 0, st, p);
        else if (kv_rank == 256) hipLaunchKernelGGL(absorb_v_kernel<2>, grid, block, 0, st, p);
        else hipLaunchKernelGGL(absorb_v_kernel<1>, grid, block, 0, st, p);
    }
    return launch_status();
}

}  // namespace dsv3
