// act_quant for gfx950: per-(1 x block) dynamic quantisation of activations to
// OCP e4m3 with one binary32 scale per block (reference: inference/kernel.py:9-35).
//
// Bandwidth-bound stream kernel.  Every lane owns 8 consecutive elements (one
// 16-byte load for bf16/fp16), so a 128-element block is one 16-lane DPP row and
// a wavefront quantises four blocks per load instruction with fully coalesced
// 1 KiB accesses.  The block amax is reduced inside the row with DPP moves, the
// scale is formed with IEEE division and the 8 quotients are converted with the
// native OCP conversion (v_cvt_pk_fp8_f32), then written as one 8-byte store.
//
// x / s is evaluated as  q0 = x*r,  e = fma(-q0, s, x),  q = fma(e, r, q0)  with
// r = RN(1/s): for bf16 x with |x| <= amax this equals the correctly rounded
// quotient wherever it can matter (every |q| >= 2^-12; below that both round to
// a zero of the same sign), which oracle/check_fast_division.c proves by
// enumeration.  Wider input types use the plain IEEE division.
#include "common.hpp"

namespace dsv3 {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 2;   // independent 16-byte loads in flight per lane (2 measured best: more costs occupancy)

template <int XD> struct In;
template <> struct In<DSV3_BF16> {
    typedef v4u vec;  // 8 x bf16
    static __device__ __forceinline__ void load(const void* p, int64_t chunk, float (&f)[8]) {
        v4u v = __builtin_nontemporal_load((const v4u*)p + chunk);
#pragma unroll
        for (int i = 0; i < 4; ++i) { f[2 * i] = bf16lo_to_f32(v[i]); f[2 * i + 1] = bf16hi_to_f32(v[i]); }
    }
};
template <> struct In<DSV3_F16> {
    static __device__ __forceinline__ void load(const void* p, int64_t chunk, float (&f)[8]) {
        v4u v = __builtin_nontemporal_load((const v4u*)p + chunk);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = v[i];
            f[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
            f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
        }
    }
};
template <> struct In<DSV3_F32> {
    static __device__ __forceinline__ void load(const void* p, int64_t chunk, float (&f)[8]) {
        v4f a = __builtin_nontemporal_load((const v4f*)p + 2 * chunk);
        v4f b = __builtin_nontemporal_load((const v4f*)p + 2 * chunk + 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) { f[i] = a[i]; f[4 + i] = b[i]; }
    }
};

// max over the LPB lanes that share a block (bit patterns of |x|, see block_scale); every lane ends with the result.
template <int LPB> __device__ __forceinline__ uint32_t group_max(uint32_t v) {
    if (LPB >= 2) v = dpp_umax<0xB1>(v);    // quad_perm [1,0,3,2]
    if (LPB >= 4) v = dpp_umax<0x4E>(v);    // quad_perm [2,3,0,1]
    if (LPB >= 8) v = dpp_umax<0x141>(v);   // row_half_mirror
    if (LPB >= 16) v = dpp_umax<0x140>(v);  // row_mirror
    if (LPB >= 32) v = umax_u32(v, (uint32_t)__shfl_xor((int)v, 16));
    if (LPB >= 64) v = umax_u32(v, (uint32_t)__shfl_xor((int)v, 32));
    return v;
}

template <int XD, int LPB, bool UE8M0>
__global__ __launch_bounds__(kThreads) void act_quant_kernel(
        const void* __restrict__ x, v2u* __restrict__ y, float* __restrict__ s, int64_t n_chunks) {
    const int64_t base = (int64_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
    float f[kUnroll][8];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t c = base + (int64_t)u * kThreads;
        if (c < n_chunks) {
            In<XD>::load(x, c, f[u]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) f[u][i] = 0.f;
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t c = base + (int64_t)u * kThreads;
        uint32_t abits = 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i) abits = umax_u32(abits, abs_bits(f[u][i]));
        abits = group_max<LPB>(abits);
        // infinity gives s = inf (finite elements quantise to 0, infinite ones to NaN), NaN gives s = NaN and a block
        // of NaN codes, in both scale formats: what the IEEE evaluation of the formula gives
        const float sc = block_scale(abits, UE8M0);
        const bool fast = XD == DSV3_BF16 && block_is_finite(abits);     // the same for all lanes of the block
        float q[8];
        if (fast) {
            const float r = 1.0f / sc;
#pragma unroll
            for (int i = 0; i < 8; ++i) q[i] = block_quotient(f[u][i], sc, r, true);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) q[i] = block_quotient(f[u][i], sc, 0.f, false);
        }
        if (c < n_chunks) {
            v2u o;
            o.x = pack_fp8x4(q[0], q[1], q[2], q[3]);
            o.y = pack_fp8x4(q[4], q[5], q[6], q[7]);
            __builtin_nontemporal_store(o, &y[c]);
            if ((c & (LPB - 1)) == 0) s[c / LPB] = sc;
        }
    }
}

template <int XD, int LPB>
int launch2(const void* x, void* y, float* s, int64_t numel, int scale_fmt, hipStream_t stream) {
    const int64_t n_chunks = numel / 8;
    const int64_t per_wg = (int64_t)kThreads * kUnroll;
    const int64_t grid = (n_chunks + per_wg - 1) / per_wg;
    if (grid > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (scale_fmt == DSV3_SCALE_FMT_UE8M0)
        hipLaunchKernelGGL((act_quant_kernel<XD, LPB, true>), dim3((unsigned)grid), dim3(kThreads), 0, stream,
                           x, (v2u*)y, s, n_chunks);
    else
        hipLaunchKernelGGL((act_quant_kernel<XD, LPB, false>), dim3((unsigned)grid), dim3(kThreads), 0, stream,
                           x, (v2u*)y, s, n_chunks);
    return launch_status();
}

// Any other block size (the reference's wrapper takes every block size that divides the last dimension,
// inference/kernel.py:38,52): one wavefront per block, the block read twice (maximum, then quotients), one element
// per lane and step.  Same arithmetic as above with the IEEE division throughout.
template <int XD> __device__ __forceinline__ float load_elem(const void* x, int64_t i) {
    if (XD == DSV3_F32) return ((const float*)x)[i];
    if (XD == DSV3_F16) return (float)((const _Float16*)x)[i];
    return u32_as_f32((uint32_t)((const uint16_t*)x)[i] << 16);
}
template <int XD>
__global__ __launch_bounds__(kThreads) void act_quant_any_block_kernel(
        const void* __restrict__ x, uint8_t* __restrict__ y, float* __restrict__ s, int64_t n_blocks, int block, int ue8m0) {
    const int lane = threadIdx.x & 63;
    const int64_t blk = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;                             // (wavefront-uniform)
    const int64_t base = blk * block;
    uint32_t abits = 0u;
    for (int i = lane; i < block; i += 64) abits = umax_u32(abits, abs_bits(load_elem<XD>(x, base + i)));
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) abits = umax_u32(abits, (uint32_t)__shfl_xor((int)abits, d));
    const float sc = block_scale(abits, ue8m0 != 0);
    for (int i = lane; i < block; i += 64) {
        const float q = load_elem<XD>(x, base + i) / sc;
        y[base + i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false) & 0xff);
    }
    if (lane == 0) s[blk] = sc;
}

template <int XD>
int launch_any_block(const void* x, void* y, float* s, int64_t numel, int block, int fmt, hipStream_t st) {
    const int64_t n_blocks = numel / block, grid = (n_blocks + kThreads / 64 - 1) / (kThreads / 64);
    if (grid > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    hipLaunchKernelGGL((act_quant_any_block_kernel<XD>), dim3((unsigned)grid), dim3(kThreads), 0, st,
                       x, (uint8_t*)y, s, n_blocks, block, fmt == DSV3_SCALE_FMT_UE8M0 ? 1 : 0);
    return launch_status();
}

template <int XD>
int launch1(const void* x, void* y, float* s, int64_t numel, int block, int fmt, hipStream_t st) {
    switch (block) {
        case 32:  return launch2<XD, 4>(x, y, s, numel, fmt, st);
        case 64:  return launch2<XD, 8>(x, y, s, numel, fmt, st);
        case 128: return launch2<XD, 16>(x, y, s, numel, fmt, st);
        case 256: return launch2<XD, 32>(x, y, s, numel, fmt, st);
        case 512: return launch2<XD, 64>(x, y, s, numel, fmt, st);
        default:  return launch_any_block<XD>(x, y, s, numel, block, fmt, st);
    }
}

}  // namespace

int launch_act_quant(const void* x, int x_dtype, void* y, float* s, int64_t numel,
                     int block_size, int scale_fmt, hipStream_t stream) {
    switch (x_dtype) {
        case DSV3_BF16: return launch1<DSV3_BF16>(x, y, s, numel, block_size, scale_fmt, stream);
        case DSV3_F16:  return launch1<DSV3_F16>(x, y, s, numel, block_size, scale_fmt, stream);
        case DSV3_F32:  return launch1<DSV3_F32>(x, y, s, numel, block_size, scale_fmt, stream);
        default: return DSV3_ERR_BAD_DTYPE;
    }
}

}  // namespace dsv3
