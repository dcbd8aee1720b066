// Shared device helpers for the gfx950 kernels: vector types, bf16/fp16/fp8
// conversions that map to single CDNA4 instructions, and launch plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <atomic>
#include "../../include/dsv3_fp8.h"

namespace dsv3 {

typedef int      v2i  __attribute__((ext_vector_type(2)));
typedef int      v4i  __attribute__((ext_vector_type(4)));
typedef int      v8i  __attribute__((ext_vector_type(8)));
typedef unsigned v2u  __attribute__((ext_vector_type(2)));
typedef unsigned v4u  __attribute__((ext_vector_type(4)));
typedef float    v2f  __attribute__((ext_vector_type(2)));
typedef float    v4f  __attribute__((ext_vector_type(4)));
typedef float    v16f __attribute__((ext_vector_type(16)));
typedef __bf16   v2bf __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

__device__ __forceinline__ float u32_as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// Two bf16 packed in a dword -> two binary32 (exact widening).
__device__ __forceinline__ float bf16lo_to_f32(uint32_t p) { return u32_as_f32(p << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t p) { return u32_as_f32(p & 0xffff0000u); }

// Two binary32 -> packed bf16, round-to-nearest-even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    v2bf r = { (__bf16)lo, (__bf16)hi };
    return __builtin_bit_cast(uint32_t, r);
}
// Two binary32 -> packed fp16, round-to-nearest-even.  The operands are made opaque first: where an FMA produces
// one of them the compiler otherwise merges the two into v_fma_mix*_f16, which rounds the exact sum straight to
// fp16 -- one rounding where every other path (and the binary32 result of the same product) has two, visible on
// results that binary32 rounds onto an fp16 tie.
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
    asm("" : "+v"(lo), "+v"(hi));
    __half2 r = __floats2half2_rn(lo, hi);
    return __builtin_bit_cast(uint32_t, r);
}

// Four binary32 -> four OCP e4m3 bytes (v_cvt_pk_fp8_f32, RNE).
__device__ __forceinline__ uint32_t pack_fp8x4(float a, float b, float c, float d) {
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
    return (uint32_t)r;
}

// e4m3 bytes of a dword -> binary32 (v_cvt_pk_f32_fp8 on the low / high half).
__device__ __forceinline__ v2f fp8x2_lo_to_f32(uint32_t p) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)p, false); }
__device__ __forceinline__ v2f fp8x2_hi_to_f32(uint32_t p) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)p, true); }

// Scale of a quantisation block (inference/kernel.py:26-31) from the largest bit pattern of |x| among its
// elements.  As unsigned integers the patterns of finite values and infinity are ordered like the values, and a NaN
// (exponent all ones, mantissa non-zero) is larger than all of them, so it reaches the scale as it does through
// torch's amax (v_max_f32 would drop it): NaN -> s = NaN, infinity -> s = inf, otherwise max(amax, 1e-4) / 448,
// rounded up to a power of two for the ue8m0 format (non-finite scales pass through unchanged).
__device__ __forceinline__ uint32_t umax_u32(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t abs_bits(float f) { return f32_as_u32(f) & 0x7fffffffu; }
// unsigned maximum of the two 16-bit halves of a and b (v_pk_max_u16)
__device__ __forceinline__ uint32_t pk_umax_u16(uint32_t a, uint32_t b) {
    typedef unsigned short v2us __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2us, a), __builtin_bit_cast(v2us, b)));
}
template <int CTRL> __device__ __forceinline__ uint32_t dpp_umax(uint32_t v) {
    return umax_u32(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ bool block_is_finite(uint32_t abits) { return abits < 0x7f800000u; }
__device__ __forceinline__ float block_scale(uint32_t abits, bool ue8m0) {
    float sc = abits > 0x7f800000u ? u32_as_f32(0x7fc00000u) : fmaxf(u32_as_f32(abits), 1e-4f) / 448.f;
    if (ue8m0 && block_is_finite(abits)) {
        const uint32_t b = f32_as_u32(sc);
        sc = u32_as_f32(((b >> 23) + ((b & 0x7fffffu) ? 1u : 0u)) << 23);
    }
    return sc;
}
// x / sc for a block element.  FAST (bf16 x of a finite block, |x| <= amax): a reciprocal and one correction step,
// equal to the correctly rounded quotient wherever the e4m3 rounding can tell (oracle/check_fast_division.c
// enumerates it); otherwise the IEEE division.
__device__ __forceinline__ float block_quotient(float x, float sc, float r, bool fast) {
    if (fast) {
        const float q0 = x * r;
        return __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-q0, sc, x), r, q0), x);
    }
    return x / sc;
}

// A binary32 value rounded to bf16 and widened again.
__device__ __forceinline__ float round_bf16(float v) { return bf16lo_to_f32(pack_bf16(v, 0.f) & 0xffffu); }

// silu(x1) * x3 as the reference's bf16 tensor operations round it (inference/model.py:633): F.silu on a bf16 tensor
// is x / (1 + exp(-x)) in binary32 rounded to bf16, then the bf16 product.  exp(-x) goes through the hardware's 2^t:
// after the rounding to bf16 the result equals the one with expf() for every bf16 x.  FAST (the caller guarantees
// |x1| < 64): the denominator is a normal number far from overflow and a reciprocal with one correction step (and x's
// sign for the zeros) rounds to the same bf16 as the IEEE division for every such x.  (Both checked on the device over
// all 65536 bf16 values; x * rcp(1 + e) without the correction differs for a few inputs, and the corrected form fails
// at x = -87.5 where the reciprocal is subnormal.)
template <bool FAST> __device__ __forceinline__ float swiglu_bf16(float x1, float x3) {
    const float d = 1.0f + __builtin_amdgcn_exp2f(-x1 * 1.44269504088896340736f);
    float sl;
    if (FAST) {
        const float r = __builtin_amdgcn_rcpf(d), q0 = x1 * r;
        sl = __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-q0, d, x1), r, q0), x1);
    } else {
        sl = x1 / d;
    }
    return round_bf16(round_bf16(sl) * x3);
}

// Output element writers: one binary32 -> C element of dsv3_dtype T.
template <int DT> struct OutT;
template <> struct OutT<DSV3_BF16> { typedef uint16_t type; static constexpr int bytes = 2; };
template <> struct OutT<DSV3_F16>  { typedef uint16_t type; static constexpr int bytes = 2; };
template <> struct OutT<DSV3_F32>  { typedef float    type; static constexpr int bytes = 4; };

template <int DT> __device__ __forceinline__ typename OutT<DT>::type cvt_out(float v);
template <> __device__ __forceinline__ uint16_t cvt_out<DSV3_BF16>(float v) { return (uint16_t)(pack_bf16(v, 0.f) & 0xffffu); }
template <> __device__ __forceinline__ uint16_t cvt_out<DSV3_F16>(float v)  { return (uint16_t)(pack_f16(v, 0.f) & 0xffffu); }
template <> __device__ __forceinline__ float    cvt_out<DSV3_F32>(float v)  { return v; }

inline int launch_status() { return hipGetLastError() == hipSuccess ? DSV3_OK : DSV3_ERR_LAUNCH; }

// More than 64 KiB of dynamic LDS has to be granted to a kernel once per device.  One LdsGrant per kernel (a
// function-local static); the per-device flags are atomics, so concurrent first calls from several threads are
// well defined (they may both make the idempotent attribute call).  Returns false when HIP refuses.
struct LdsGrant {
    std::atomic<bool> done[64];
    bool ensure(const void* kernel, int bytes) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
        if (done[dev].load(std::memory_order_acquire)) return true;
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
        done[dev].store(true, std::memory_order_release);
        return true;
    }
};

// Entry points of the individual kernel families (defined in the .hip files).
int launch_act_quant(const void* x, int x_dtype, void* y, float* s, int64_t numel,
                     int block_size, int scale_fmt, hipStream_t stream);
int launch_weight_dequant(const void* x, const float* s, void* y, int y_dtype,
                          int64_t m, int64_t n, int block_size, hipStream_t stream);
int launch_weight_quant(const void* w, int w_dtype, void* y, float* s, int64_t m, int64_t n, int scale_fmt,
                        hipStream_t stream);
int launch_fp8_gemm(const void* a, const float* a_s, const void* b, const float* b_s,
                    void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                    void* workspace, size_t workspace_bytes, hipStream_t stream, bool pow2_scales = false);
size_t fp8_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k);
bool prefill_supported(int64_t m, int64_t n, int64_t k);
bool stream_supported(int64_t m, int64_t n, int64_t k);
size_t stream_workspace_bytes(int64_t m, int64_t n, int64_t k);
int launch_stream(const void* a, const float* a_s, const void* b, const float* b_s, void* c, int c_dtype,
                  int64_t m, int64_t n, int64_t k, void* ws, int* splits_out, hipStream_t st);
bool skinny_supported(int64_t m, int64_t n, int64_t k);
size_t skinny_workspace_bytes(int64_t m, int64_t n, int64_t k);
int launch_skinny(const void* a, const float* a_s, const void* b, const float* b_s, void* c, int c_dtype,
                  int64_t m, int64_t n, int64_t k, void* ws, int* splits_out, hipStream_t st, int quant_mode = 0);
int launch_linear_fp8(const void* x, const void* b, const float* b_s, void* c, int c_dtype, int64_t m, int64_t n,
                      int64_t k, int scale_fmt, void* workspace, hipStream_t stream);
bool linear_fp8_supported(int64_t m, int64_t n, int64_t k);
size_t prefill_workspace_bytes(int64_t m, int64_t n, int64_t k);
template <int CD, bool P2 = false>        // P2: every scale is a power of two (they go into the MFMA's scale operands)
int launch_prefill(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                   int64_t m, int64_t n, int64_t k, void* ws, hipStream_t stream);
int grouped_tile_rows();
bool grouped_supported(int64_t a_num_rows, int64_t n, int64_t k);
template <int CD, bool P2 = false>
int launch_grouped(const void* a, const float* a_s, const int* a_rows, const void* b, const float* b_s, void* c,
                   int64_t m, int64_t n, int64_t k, int64_t num_tiles, const int* tile_group, const int* tile_row0,
                   const int* tile_rows, int64_t b_stride, int64_t bs_stride, hipStream_t stream);
bool grouped_swiglu_supported(int64_t m, int64_t a_num_rows, int64_t inter, int64_t k);
int launch_grouped_swiglu(const void* a, const float* a_s, const int* a_rows, const void* b, const float* b_s,
                          void* y, float* s, int64_t m, int64_t inter, int64_t k, int64_t num_tiles,
                          const int* tile_group, const int* tile_row0, const int* tile_rows, int64_t b_stride,
                          int64_t bs_stride, int scale_fmt, hipStream_t stream);
int launch_grouped_skinny(const void* a, const float* a_s, const int* a_rows, const void* b, const float* b_s, void* c,
                          int c_dtype, int64_t n, int64_t k, int64_t num_tiles, const int* tile_group,
                          const int* tile_row0, const int* tile_rows, int64_t b_stride, int64_t bs_stride,
                          int64_t groups_hint, hipStream_t stream);
bool skinny_single_supported(int64_t m, int64_t n, int64_t k);
int launch_skinny_single(const void* a, const float* a_s, const void* b, const float* b_s, void* c, int c_dtype,
                         int64_t m, int64_t n, int64_t k, hipStream_t stream);
int launch_swiglu_quant(const void* h, void* y, float* s, int64_t rows, int64_t inter, int scale_fmt, hipStream_t st);
int launch_moe_combine(const void* out, const int* rows, const void* w, const void* shared, void* y,
                       int64_t tokens, int topk, int64_t dim, hipStream_t st);
int launch_moe_route(const int64_t* indices, const void* weights, int64_t tokens, int topk, int experts,
                     int shared_one, int max_tiles, int tile_rows, int* counts, int* offsets, int* cursor, int* a_rows,
                     int* rows, void* w_sorted, int* tile_group, int* tile_row0, int* tile_nrows, hipStream_t st);
int launch_group_tiles(const int* counts, int groups, int tile_rows, int max_tiles,
                       int* tile_group, int* tile_row0, int* tile_nrows, hipStream_t st);
int launch_gate_route(const void* logits, const float* bias, void* weights, int64_t* indices, int64_t tokens,
                      int experts, int topk, int n_groups, int topk_groups, int score_func, float route_scale,
                      hipStream_t st);
bool wkv_b_absorb_supported(int side, int nope, int v, int64_t kv_rank);
int launch_wkv_b_absorb(const void* x, int64_t x_ts, int64_t x_hs, const void* w, const float* ws, void* y, int side,
                        int64_t tokens, int heads, int nope, int v, int64_t kv_rank, hipStream_t st);

}  // namespace dsv3
