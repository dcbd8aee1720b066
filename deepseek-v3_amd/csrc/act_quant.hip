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

// The block maximum is taken over the bit patterns of |x| as unsigned integers: for finite values and infinity that
// is the order of the values, and a NaN (exponent all ones, mantissa non-zero) is larger than everything, so it
// reaches the scale the way torch's amax and the reference's tl.max let it (v_max_f32 would drop it).
__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }
template <int CTRL> __device__ __forceinline__ uint32_t dpp_max(uint32_t v) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
    return umax(v, o);
}

// max over the LPB lanes that share a block; every lane ends with the result.
template <int LPB> __device__ __forceinline__ uint32_t group_max(uint32_t v) {
    if (LPB >= 2) v = dpp_max<0xB1>(v);    // quad_perm [1,0,3,2]
    if (LPB >= 4) v = dpp_max<0x4E>(v);    // quad_perm [2,3,0,1]
    if (LPB >= 8) v = dpp_max<0x141>(v);   // row_half_mirror
    if (LPB >= 16) v = dpp_max<0x140>(v);  // row_mirror
    if (LPB >= 32) v = umax(v, (uint32_t)__shfl_xor((int)v, 16));
    if (LPB >= 64) v = umax(v, (uint32_t)__shfl_xor((int)v, 32));
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
        for (int i = 0; i < 8; ++i) abits = umax(abits, f32_as_u32(f[u][i]) & 0x7fffffffu);
        abits = group_max<LPB>(abits);
        const bool finite = abits < 0x7f800000u;                 // the same for all lanes of the block
        // infinity gives s = inf (finite elements quantise to 0, infinite ones to NaN), NaN gives s = NaN and a block
        // of NaN codes: what the IEEE evaluation of the formula gives
        float sc = abits > 0x7f800000u ? u32_as_f32(0x7fc00000u) : fmaxf(u32_as_f32(abits), 1e-4f) / 448.f;
        if (UE8M0) {
            uint32_t b = f32_as_u32(sc);
            b = ((b >> 23) + ((b & 0x7fffffu) ? 1u : 0u)) << 23;
            sc = u32_as_f32(b);
        }
        float q[8];
        if (XD == DSV3_BF16 && finite) {
            const float r = 1.0f / sc;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float q0 = f[u][i] * r;
                const float e = __builtin_fmaf(-q0, sc, f[u][i]);
                q[i] = __builtin_copysignf(__builtin_fmaf(e, r, q0), f[u][i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) q[i] = f[u][i] / sc;
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

template <int XD>
int launch1(const void* x, void* y, float* s, int64_t numel, int block, int fmt, hipStream_t st) {
    switch (block) {
        case 32:  return launch2<XD, 4>(x, y, s, numel, fmt, st);
        case 64:  return launch2<XD, 8>(x, y, s, numel, fmt, st);
        case 128: return launch2<XD, 16>(x, y, s, numel, fmt, st);
        case 256: return launch2<XD, 32>(x, y, s, numel, fmt, st);
        case 512: return launch2<XD, 64>(x, y, s, numel, fmt, st);
        default:  return DSV3_ERR_BAD_BLOCK;
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
