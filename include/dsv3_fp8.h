/*
 * dsv3_fp8.h -- C ABI of libdsv3fp8.so: DeepSeek-V3's block-scaled FP8 inference
 * kernels, written for AMD MI355X (gfx950).
 *
 * The three compute entry points replace, one for one, the three Python
 * functions of the reference's inference/kernel.py (the only callers are
 * inference/model.py:156-160, :481 and inference/fp8_cast_bf16.py:80):
 *
 *   dsv3_act_quant       <- act_quant       (inference/kernel.py:38-57,  kernel :9-35)
 *   dsv3_weight_dequant  <- weight_dequant  (inference/kernel.py:89-110, kernel :60-86)
 *   dsv3_fp8_gemm        <- fp8_gemm        (inference/kernel.py:175-196, kernel :118-172)
 *
 * Conventions
 *   - every pointer is a device pointer into memory the caller owns; the library
 *     never allocates, frees or keeps caller-visible memory;
 *   - work is enqueued on `stream` (a hipStream_t; NULL = the null stream) and the
 *     call returns without synchronising;
 *   - every function returns a dsv3_status; arguments are validated on the host
 *     before any GPU call is made, so the error paths work on a machine with no GPU;
 *   - "fp8" is OCP E4M3 (torch.float8_e4m3fn); scales are IEEE binary32;
 *   - tensors are dense and row-major ("contiguous" in the reference's asserts,
 *     inference/kernel.py:51, :104, :188-189).
 */
#ifndef DSV3_FP8_H
#define DSV3_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum dsv3_status {
    DSV3_OK = 0,
    DSV3_ERR_NULL_POINTER = 1,  /* a required pointer is NULL                              */
    DSV3_ERR_BAD_SHAPE = 2,     /* negative size, or last dim not a multiple of the block */
    DSV3_ERR_BAD_BLOCK = 3,     /* block size the kernels do not implement                 */
    DSV3_ERR_MISALIGNED = 4,    /* pointer not aligned as documented                       */
    DSV3_ERR_BAD_DTYPE = 5,     /* dtype code not in dsv3_dtype / not valid here           */
    DSV3_ERR_WORKSPACE = 6,     /* workspace missing or smaller than the size query says   */
    DSV3_ERR_LAUNCH = 7         /* HIP reported an error at launch                         */
} dsv3_status;

typedef enum dsv3_dtype {
    DSV3_BF16 = 0,
    DSV3_F16 = 1,
    DSV3_F32 = 2
} dsv3_dtype;

/* scale_fmt of act_quant (inference/kernel.py:29-31): NONE keeps s = amax/448,
 * UE8M0 rounds s up to a power of two. */
typedef enum dsv3_scale_fmt {
    DSV3_SCALE_FMT_NONE = 0,
    DSV3_SCALE_FMT_UE8M0 = 1
} dsv3_scale_fmt;

/* Library version: major*10000 + minor*100 + patch. */
int dsv3_version(void);

/* Static, NUL-terminated description of a dsv3_status (never NULL). */
const char* dsv3_status_string(int status);

/*
 * act_quant (inference/kernel.py:23-35).  For each run of `block_size`
 * contiguous elements of x:
 *     amax = max|x|;  amax = max(amax, 1e-4f);  s = amax / 448.f;
 *     if scale_fmt == UE8M0:  s = 2^ceil(log2 s);
 *     y = e4m3( f32(x) / s )            (IEEE division, round-to-nearest-even)
 * x: [numel] of x_dtype, y: [numel] bytes, s: [numel / block_size] binary32.
 * `last_dim` is x.size(-1); it must be a multiple of block_size (the reference's
 * assert at inference/kernel.py:52) and numel a multiple of last_dim.
 * block_size in {32, 64, 128, 256, 512}.  x and y must be 16-byte aligned.
 * numel == 0 is a no-op.  The result is bit-identical to the IEEE evaluation of
 * the formula above for finite inputs.
 */
int dsv3_act_quant(const void* x, int x_dtype, void* y, float* s,
                   int64_t numel, int64_t last_dim, int block_size,
                   int scale_fmt, void* stream);

/*
 * weight_dequant (inference/kernel.py:76-86):
 *     y[i,j] = y_dtype( f32(x[i,j]) * s[i / block_size, j / block_size] )
 * x: [m,n] fp8 bytes, s: [ceil(m/block_size), ceil(n/block_size)] binary32,
 * y: [m,n] of y_dtype.  Any m, n >= 0 and any block_size >= 1; block_size 128
 * with n % 8 == 0, 8-byte aligned x and 16-byte aligned y takes the vectorised kernel.
 */
int dsv3_weight_dequant(const void* x, const float* s, void* y, int y_dtype,
                        int64_t m, int64_t n, int block_size, void* stream);

/*
 * fp8_gemm (inference/kernel.py:145-172):
 *     c[i,j] = c_dtype( sum_kb ( sum_{t<128} a[i,128kb+t] * b[j,128kb+t] )
 *                                * a_s[i,kb] * b_s[j/128,kb] )
 * a: [m,k] fp8, a_s: [m,k/128] binary32, b: [n,k] fp8 (the weight, out x in),
 * b_s: [ceil(n/128), k/128] binary32, c: [m,n] of c_dtype.  Products and sums
 * are binary32; the order of additions differs from the reference's.
 * k must be a multiple of 128 (guaranteed by act_quant, inference/kernel.py:52);
 * any m, n >= 0.  a and b must be 16-byte aligned.
 * `workspace` must hold at least dsv3_fp8_gemm_workspace_bytes(m,n,k) bytes
 * (256-byte aligned) when that is non-zero; its contents on entry are ignored
 * and are undefined on return.  Calls sharing a workspace must be ordered on
 * one stream.
 */
int dsv3_fp8_gemm(const void* a, const float* a_s, const void* b, const float* b_s,
                  void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                  void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of scratch dsv3_fp8_gemm needs for this problem (0 when none). */
size_t dsv3_fp8_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k);

#ifdef __cplusplus
}
#endif
#endif /* DSV3_FP8_H */
