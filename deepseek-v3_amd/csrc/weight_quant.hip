// weight_quant for gfx950: per-(128 x 128) block quantisation of a weight matrix to OCP e4m3 with one binary32
// scale per block -- the inverse of weight_dequant and the producer of the on-disk format the reference reads
// (README_WEIGHTS.md:60-92: `weight` + `weight_scale_inv`, 128 x 128 blocks, a ragged block is zero-padded before
// its scale is taken and cropped afterwards; scale tensor shape inference/model.py:184-187).
//
//     s[i,j] = max(amax(block i,j), 1e-4) / 448        w8 = e4m3( w / s[i,j] )        so that  w ~= w8 * s
// (scale_fmt ue8m0: s rounded up to a power of two first, the format of checkpoints made for
// inference/configs/config_v3.1.json:22)
//
// the arithmetic of act_quant (inference/kernel.py:23-35) applied to a square block: amax, the clamp that keeps an
// all-zero block finite, an IEEE division by 448, a correctly rounded quotient, round-to-nearest-even to e4m3.
//
// Bandwidth-bound.  One workgroup of 256 threads owns one block: 16 lanes cover the 128 columns of a row (16-byte
// loads of 8 bf16, 256 contiguous bytes per row and 4 rows per wavefront instruction), a thread holds 8 rows x 8
// columns in registers -- the block is read once --, the amax goes through DPP (row), two lane exchanges
// (wavefront) and LDS (4 wavefronts), and every thread then writes 8 bytes per row it holds.
//
// w / s for bf16 w uses the same reciprocal-and-correction sequence as act_quant (see act_quant.hip: exact wherever
// the e4m3 rounding can see a difference, for |w| <= amax); wider inputs use the IEEE division.
#include <type_traits>
#include "common.hpp"

namespace dsv3 {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerThread = 8;      // rows r0 + 16 i of the block

template <int XD> __device__ __forceinline__ float load_one(const void* p, int64_t i);
template <> __device__ __forceinline__ float load_one<DSV3_BF16>(const void* p, int64_t i) {
    return u32_as_f32((uint32_t)((const uint16_t*)p)[i] << 16);
}
template <> __device__ __forceinline__ float load_one<DSV3_F16>(const void* p, int64_t i) {
    return (float)__builtin_bit_cast(_Float16, ((const uint16_t*)p)[i]);
}
template <> __device__ __forceinline__ float load_one<DSV3_F32>(const void* p, int64_t i) { return ((const float*)p)[i]; }

// 8 consecutive elements starting at element index i (a multiple of 8, 16-byte aligned for the 2-byte types)
template <int XD> __device__ __forceinline__ void load8(const void* p, int64_t i, float (&f)[8]) {
    if (XD == DSV3_F32) {
        const v4f a = __builtin_nontemporal_load((const v4f*)((const float*)p + i));
        const v4f b = __builtin_nontemporal_load((const v4f*)((const float*)p + i) + 1);
#pragma unroll
        for (int e = 0; e < 4; ++e) { f[e] = a[e]; f[4 + e] = b[e]; }
    } else {
        const v4u v = __builtin_nontemporal_load((const v4u*)((const uint16_t*)p + i));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (XD == DSV3_BF16) {
                f[2 * e] = bf16lo_to_f32(v[e]);
                f[2 * e + 1] = bf16hi_to_f32(v[e]);
            } else {
                f[2 * e] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[e] & 0xffffu));
                f[2 * e + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[e] >> 16));
            }
        }
    }
}

// VEC: n % 8 == 0 and 16-byte aligned bases, so an 8-element chunk is loaded and stored whole and lies entirely
// inside or outside the matrix; otherwise every element is guarded on its own.
template <int XD, bool VEC>
__global__ __launch_bounds__(kThreads) void weight_quant_kernel(
        const void* __restrict__ w, uint8_t* __restrict__ y, float* __restrict__ s, int m, int n, int nb, int ue8m0) {
    __shared__ uint32_t wave_max[kThreads / kWave];
    const int t = threadIdx.x;
    const int col = blockIdx.x * 128 + (t & 15) * 8;           // first of the thread's 8 columns
    const int row0 = blockIdx.y * 128 + (t >> 4);              // its rows: row0 + 16 i

    float f[kRowsPerThread][8];
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int row = row0 + 16 * i;
        const int64_t at = (int64_t)row * n + col;
        if (VEC) {
            if (row < m && col < n) {
                load8<XD>(w, at, f[i]);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) f[i][e] = 0.f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) f[i][e] = (row < m && col + e < n) ? load_one<XD>(w, at + e) : 0.f;
        }
    }

    uint32_t abits = 0u;                       // non-finite values reach the scale as in act_quant
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) abits = umax_u32(abits, abs_bits(f[i][e]));
    abits = dpp_umax<0xB1>(abits);             // quad_perm [1,0,3,2]
    abits = dpp_umax<0x4E>(abits);             // quad_perm [2,3,0,1]
    abits = dpp_umax<0x141>(abits);            // row_half_mirror
    abits = dpp_umax<0x140>(abits);            // row_mirror: the 16 lanes of a DPP row agree
    abits = umax_u32(abits, (uint32_t)__shfl_xor((int)abits, 16));
    abits = umax_u32(abits, (uint32_t)__shfl_xor((int)abits, 32));
    if ((t & 63) == 0) wave_max[t >> 6] = abits;
    __syncthreads();
    abits = umax_u32(umax_u32(wave_max[0], wave_max[1]), umax_u32(wave_max[2], wave_max[3]));
    // (ue8m0: the scale rounded up to a power of two, as act_quant does, kernel.py:29-31)
    const float sc = block_scale(abits, ue8m0 != 0);
    const bool fast = XD == DSV3_BF16 && block_is_finite(abits);
    if (t == 0) s[(int64_t)blockIdx.y * nb + blockIdx.x] = sc;

    // (a workgroup-uniform branch around the whole write-out: one of the two division sequences is executed)
    auto write_out = [&](auto fast_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
        const float r = FAST ? 1.0f / sc : 0.f;
#pragma unroll
        for (int i = 0; i < kRowsPerThread; ++i) {
            const int row = row0 + 16 * i;
            float q[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) q[e] = block_quotient(f[i][e], sc, r, FAST);
            const v2u o = { pack_fp8x4(q[0], q[1], q[2], q[3]), pack_fp8x4(q[4], q[5], q[6], q[7]) };
            const int64_t at = (int64_t)row * n + col;
            if (VEC) {
                if (row < m && col < n) __builtin_nontemporal_store(o, (v2u*)(y + at));
            } else if (row < m) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (col + e < n) y[at + e] = (uint8_t)((o[e >> 2] >> (8 * (e & 3))) & 0xffu);
            }
        }
    };
    if (fast) write_out(std::true_type{});
    else      write_out(std::false_type{});
}

template <int XD>
int launch1(const void* w, void* y, float* s, int64_t m, int64_t n, int ue8m0, hipStream_t stream) {
    const int64_t mb = (m + 127) / 128, nb = (n + 127) / 128;
    if (mb > 65535 || nb > 0x7fffffff || m > 0x7fffffff || n > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    const bool vec = (n % 8) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)y % 8) == 0;
    const dim3 grid((unsigned)nb, (unsigned)mb);
    if (vec)
        hipLaunchKernelGGL((weight_quant_kernel<XD, true>), grid, dim3(kThreads), 0, stream, w, (uint8_t*)y, s,
                           (int)m, (int)n, (int)nb, ue8m0);
    else
        hipLaunchKernelGGL((weight_quant_kernel<XD, false>), grid, dim3(kThreads), 0, stream, w, (uint8_t*)y, s,
                           (int)m, (int)n, (int)nb, ue8m0);
    return launch_status();
}

}  // namespace

int launch_weight_quant(const void* w, int w_dtype, void* y, float* s, int64_t m, int64_t n, int scale_fmt,
                        hipStream_t stream) {
    const int ue8m0 = scale_fmt == DSV3_SCALE_FMT_UE8M0;
    switch (w_dtype) {
        case DSV3_BF16: return launch1<DSV3_BF16>(w, y, s, m, n, ue8m0, stream);
        case DSV3_F16:  return launch1<DSV3_F16>(w, y, s, m, n, ue8m0, stream);
        case DSV3_F32:  return launch1<DSV3_F32>(w, y, s, m, n, ue8m0, stream);
        default: return DSV3_ERR_BAD_DTYPE;
    }
}

}  // namespace dsv3
