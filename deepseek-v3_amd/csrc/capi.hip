// C ABI of libdsv3fp8.so: host-side argument validation and dispatch.
// Everything is checked before the first HIP call so that the error paths are
// usable (and tested) on a machine without a GPU.
#include <mutex>
#include "common.hpp"

using namespace dsv3;

// Split-K scratch of dsv3_fp8_gemm_static: part of the loaded code object, so every GPU the library runs on holds
// its own copy at its own address until the process ends.  Host code never passes this name to a kernel (on the
// host it is only a stand-in for the symbol): static_scratch() resolves the device address once per device.
static __device__ __align__(256) unsigned char scratch[DSV3_STATIC_SCRATCH_BYTES];

namespace {
inline bool aligned(const void* p, uintptr_t a) { return ((uintptr_t)p % a) == 0; }
inline bool valid_dtype(int d) { return d == DSV3_BF16 || d == DSV3_F16 || d == DSV3_F32; }

// Device address of `scratch` on the current device (nullptr on failure); resolved on the first call per device.
void* static_scratch() {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* ptr[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return nullptr;
        }
        ptr[dev] = p;
    }
    return ptr[dev];
}
}

extern "C" {

int dsv3_version(void) { return 100; }

const char* dsv3_status_string(int status) {
    switch (status) {
        case DSV3_OK: return "ok";
        case DSV3_ERR_NULL_POINTER: return "null pointer";
        case DSV3_ERR_BAD_SHAPE: return "bad shape (negative size, or last dimension not a multiple of the block size)";
        case DSV3_ERR_BAD_BLOCK: return "unsupported block size";
        case DSV3_ERR_MISALIGNED: return "pointer not aligned as required";
        case DSV3_ERR_BAD_DTYPE: return "unsupported dtype code";
        case DSV3_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case DSV3_ERR_LAUNCH: return "HIP launch failed";
        case DSV3_ERR_TOO_LARGE: return "problem needs more scratch than the library's fixed array holds (use the entry point that takes a workspace)";
        default: return "unknown status";
    }
}

int dsv3_act_quant(const void* x, int x_dtype, void* y, float* s,
                   int64_t numel, int64_t last_dim, int block_size,
                   int scale_fmt, void* stream) {
    if (!valid_dtype(x_dtype)) return DSV3_ERR_BAD_DTYPE;
    if (scale_fmt != DSV3_SCALE_FMT_NONE && scale_fmt != DSV3_SCALE_FMT_UE8M0) return DSV3_ERR_BAD_DTYPE;
    if (block_size < 1) return DSV3_ERR_BAD_BLOCK;
    if (numel < 0 || last_dim < 0) return DSV3_ERR_BAD_SHAPE;
    if (last_dim % block_size != 0) return DSV3_ERR_BAD_SHAPE;
    if (numel == 0) return DSV3_OK;
    if (last_dim == 0 || numel % last_dim != 0) return DSV3_ERR_BAD_SHAPE;
    if (!x || !y || !s) return DSV3_ERR_NULL_POINTER;
    if (!aligned(x, 16) || !aligned(y, 8) || !aligned(s, 4)) return DSV3_ERR_MISALIGNED;
    return launch_act_quant(x, x_dtype, y, s, numel, block_size, scale_fmt, (hipStream_t)stream);
}

int dsv3_weight_dequant(const void* x, const float* s, void* y, int y_dtype,
                        int64_t m, int64_t n, int block_size, void* stream) {
    if (!valid_dtype(y_dtype)) return DSV3_ERR_BAD_DTYPE;
    if (block_size < 1) return DSV3_ERR_BAD_BLOCK;
    if (m < 0 || n < 0) return DSV3_ERR_BAD_SHAPE;
    if (m == 0 || n == 0) return DSV3_OK;
    if (!x || !s || !y) return DSV3_ERR_NULL_POINTER;
    if (!aligned(s, 4) || !aligned(y, y_dtype == DSV3_F32 ? 4 : 2)) return DSV3_ERR_MISALIGNED;
    return launch_weight_dequant(x, s, y, y_dtype, m, n, block_size, (hipStream_t)stream);
}

int dsv3_weight_quant(const void* w, int w_dtype, void* y, float* s,
                      int64_t m, int64_t n, int block_size, int scale_fmt, void* stream) {
    if (!valid_dtype(w_dtype)) return DSV3_ERR_BAD_DTYPE;
    if (scale_fmt != DSV3_SCALE_FMT_NONE && scale_fmt != DSV3_SCALE_FMT_UE8M0) return DSV3_ERR_BAD_DTYPE;
    if (block_size != 128) return DSV3_ERR_BAD_BLOCK;
    if (m < 0 || n < 0) return DSV3_ERR_BAD_SHAPE;
    if (m == 0 || n == 0) return DSV3_OK;
    if (!w || !y || !s) return DSV3_ERR_NULL_POINTER;
    if (!aligned(s, 4) || !aligned(w, w_dtype == DSV3_F32 ? 4 : 2)) return DSV3_ERR_MISALIGNED;
    return launch_weight_quant(w, w_dtype, y, s, m, n, scale_fmt, (hipStream_t)stream);
}

size_t dsv3_fp8_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || n <= 0 || k <= 0 || k % 128 != 0) return 0;
    return fp8_gemm_workspace_bytes(m, n, k);
}

// Host-side checks of the fp8_gemm entry points (no GPU call).  DSV3_OK with m == 0 or n == 0 means "nothing to do".
static int fp8_gemm_validate(const void* a, const float* a_s, const void* b, const float* b_s,
                             void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                             void* workspace, size_t workspace_bytes, bool check_workspace = true) {
    if (!valid_dtype(c_dtype)) return DSV3_ERR_BAD_DTYPE;
    if (m < 0 || n < 0 || k < 0) return DSV3_ERR_BAD_SHAPE;
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    // (K need not be a multiple of 128: the last block is then masked, as in the reference's kernel; m is a grid
    // dimension of that fallback)
    if (k % 128 != 0 && m > 65535) return DSV3_ERR_BAD_SHAPE;
    if (m == 0 || n == 0) return DSV3_OK;
    if (!c) return DSV3_ERR_NULL_POINTER;
    if (k > 0 && (!a || !a_s || !b || !b_s)) return DSV3_ERR_NULL_POINTER;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(a_s, 4) || !aligned(b_s, 4) ||
        !aligned(c, c_dtype == DSV3_F32 ? 16 : 8))
        return DSV3_ERR_MISALIGNED;
    if (!check_workspace) return DSV3_OK;
    const size_t need = dsv3_fp8_gemm_workspace_bytes(m, n, k);
    if (need > 0 && (!workspace || workspace_bytes < need || !aligned(workspace, 256))) return DSV3_ERR_WORKSPACE;
    return DSV3_OK;
}

static int fp8_gemm_checked(const void* a, const float* a_s, const void* b, const float* b_s,
                           void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                           void* workspace, size_t workspace_bytes, void* stream, bool pow2_scales) {
    const int rc = fp8_gemm_validate(a, a_s, b, b_s, c, c_dtype, m, n, k, workspace, workspace_bytes);
    if (rc != DSV3_OK || m == 0 || n == 0) return rc;
    return launch_fp8_gemm(a, a_s, b, b_s, c, c_dtype, m, n, k, workspace, workspace_bytes, (hipStream_t)stream,
                           pow2_scales);
}

int dsv3_fp8_gemm(const void* a, const float* a_s, const void* b, const float* b_s,
                  void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                  void* workspace, size_t workspace_bytes, void* stream) {
    return fp8_gemm_checked(a, a_s, b, b_s, c, c_dtype, m, n, k, workspace, workspace_bytes, stream, false);
}

int dsv3_fp8_gemm_pow2(const void* a, const float* a_s, const void* b, const float* b_s,
                       void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                       void* workspace, size_t workspace_bytes, void* stream) {
    return fp8_gemm_checked(a, a_s, b, b_s, c, c_dtype, m, n, k, workspace, workspace_bytes, stream, true);
}

size_t dsv3_fp8_gemm_static_max_bytes(void) { return DSV3_STATIC_SCRATCH_BYTES; }

int dsv3_fp8_gemm_static(const void* a, const float* a_s, const void* b, const float* b_s,
                         void* c, int c_dtype, int64_t m, int64_t n, int64_t k, void* stream) {
    // the argument checks of dsv3_fp8_gemm first (no GPU call on an error path), then the size of the scratch: a
    // malformed call reports what is wrong with it, not DSV3_ERR_TOO_LARGE
    const int rc = fp8_gemm_validate(a, a_s, b, b_s, c, c_dtype, m, n, k, nullptr, 0, false);
    if (rc != DSV3_OK || m == 0 || n == 0) return rc;
    const size_t need = dsv3_fp8_gemm_workspace_bytes(m, n, k);
    if (need > DSV3_STATIC_SCRATCH_BYTES) return DSV3_ERR_TOO_LARGE;     // refused before anything is launched
    void* ws = nullptr;
    if (need) {
        ws = static_scratch();
        if (!ws) return DSV3_ERR_LAUNCH;
    }
    return launch_fp8_gemm(a, a_s, b, b_s, c, c_dtype, m, n, k, ws, DSV3_STATIC_SCRATCH_BYTES, (hipStream_t)stream, false);
}

int dsv3_linear_fp8_fused(int64_t m, int64_t n, int64_t k) {
    return m > 0 && n > 0 && k > 0 && m <= 0x7fffffff && n <= 0x7fffffff && k <= 0x7fffffff && linear_fp8_supported(m, n, k);
}

int dsv3_linear_fp8(const void* x, int x_dtype, const void* b, const float* b_s, void* c, int c_dtype,
                    int64_t m, int64_t n, int64_t k, int block_size, int scale_fmt,
                    void* workspace, size_t workspace_bytes, void* stream) {
    if (x_dtype != DSV3_BF16 || !valid_dtype(c_dtype)) return DSV3_ERR_BAD_DTYPE;
    if (scale_fmt != DSV3_SCALE_FMT_NONE && scale_fmt != DSV3_SCALE_FMT_UE8M0) return DSV3_ERR_BAD_DTYPE;
    if (block_size != 128) return DSV3_ERR_BAD_BLOCK;
    if (m < 0 || n < 0 || k < 0 || k % 128 != 0) return DSV3_ERR_BAD_SHAPE;
    if (m == 0 || n == 0) return DSV3_OK;
    if (!dsv3_linear_fp8_fused(m, n, k)) return DSV3_ERR_BAD_SHAPE;       // ask dsv3_linear_fp8_fused first
    if (!x || !b || !b_s || !c) return DSV3_ERR_NULL_POINTER;
    if (!aligned(x, 16) || !aligned(b, 16) || !aligned(b_s, 4) || !aligned(c, c_dtype == DSV3_F32 ? 16 : 8))
        return DSV3_ERR_MISALIGNED;
    const size_t need = dsv3_fp8_gemm_workspace_bytes(m, n, k);
    if (need > 0 && (!workspace || workspace_bytes < need || !aligned(workspace, 256))) return DSV3_ERR_WORKSPACE;
    return launch_linear_fp8(x, b, b_s, c, c_dtype, m, n, k, scale_fmt, workspace, (hipStream_t)stream);
}

int dsv3_fp8_gemm_grouped_tile_rows(void) { return grouped_tile_rows(); }

int dsv3_group_tiles(const int32_t* counts, int groups, int max_tiles,
                     int32_t* tile_group, int32_t* tile_row0, int32_t* tile_rows, void* stream) {
    if (groups < 0 || max_tiles < 0) return DSV3_ERR_BAD_SHAPE;
    if (max_tiles == 0) return DSV3_OK;
    if ((groups > 0 && !counts) || !tile_group || !tile_row0 || !tile_rows) return DSV3_ERR_NULL_POINTER;
    return launch_group_tiles(counts, groups, grouped_tile_rows(), max_tiles, tile_group, tile_row0, tile_rows,
                              (hipStream_t)stream);
}

int dsv3_moe_route(const int64_t* indices, const void* weights, int w_dtype, int64_t tokens, int topk, int experts,
                   int shared_group, int max_tiles, int32_t* scratch, int32_t* a_rows, int32_t* rows, void* w_sorted,
                   int32_t* tile_group, int32_t* tile_row0, int32_t* tile_rows, void* stream) {
    if (w_dtype != DSV3_BF16 && w_dtype != DSV3_F16) return DSV3_ERR_BAD_DTYPE;       // any 2-byte type: values are only moved
    if (tokens < 0 || topk < 1 || topk > 16 || experts < 1 || experts > 8192 || max_tiles < 0) return DSV3_ERR_BAD_SHAPE;
    if (tokens * (topk + 1) > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (!scratch || (max_tiles > 0 && (!tile_group || !tile_row0 || !tile_rows))) return DSV3_ERR_NULL_POINTER;
    if (tokens > 0 && (!indices || !weights || !a_rows || !rows || !w_sorted)) return DSV3_ERR_NULL_POINTER;
    if (!aligned(indices, 8) || !aligned(weights, 2) || !aligned(w_sorted, 2)) return DSV3_ERR_MISALIGNED;
    const int groups = experts + (shared_group ? 1 : 0);
    const int one = shared_group ? (w_dtype == DSV3_BF16 ? 0x3F80 : 0x3C00) : 0;     // 1.0 in the weights' type
    return launch_moe_route(indices, weights, tokens, topk, experts, one, max_tiles, grouped_tile_rows(),
                            scratch, scratch + groups, scratch + 2 * (int64_t)groups, a_rows, rows, w_sorted,
                            tile_group, tile_row0, tile_rows, (hipStream_t)stream);
}

static int fp8_gemm_grouped_checked(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                                   const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                                   void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                                   const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                                   int64_t num_tiles, void* stream, bool pow2) {
    if (!valid_dtype(c_dtype)) return DSV3_ERR_BAD_DTYPE;
    if (m < 0 || n < 0 || k < 0 || a_num_rows < 0 || num_tiles < 0 || b_group_stride < 0 || bs_group_stride < 0)
        return DSV3_ERR_BAD_SHAPE;
    if (k % 128 != 0 || k == 0) return DSV3_ERR_BAD_SHAPE;
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (m == 0 || n == 0 || num_tiles == 0) return DSV3_OK;
    if (!a || !a_s || !b || !b_s || !c || !tile_group || !tile_row0 || !tile_rows) return DSV3_ERR_NULL_POINTER;
    if (!aligned(a, 16) || !aligned(b, 16) || b_group_stride % 16 != 0 || !aligned(a_s, 4) || !aligned(b_s, 4) ||
        !aligned(c, c_dtype == DSV3_F32 ? 16 : 8))
        return DSV3_ERR_MISALIGNED;
    if (!grouped_supported(a_num_rows, n, k)) return DSV3_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
#define DSV3_GROUPED(CD)                                                                                              \
    (pow2 ? launch_grouped<CD, true>(a, a_s, a_rows, b, b_s, c, m, n, k, num_tiles, tile_group, tile_row0, tile_rows,  \
                                     b_group_stride, bs_group_stride, st)                                              \
          : launch_grouped<CD, false>(a, a_s, a_rows, b, b_s, c, m, n, k, num_tiles, tile_group, tile_row0, tile_rows, \
                                      b_group_stride, bs_group_stride, st))
    switch (c_dtype) {
        case DSV3_BF16: return DSV3_GROUPED(DSV3_BF16);
        case DSV3_F16:  return DSV3_GROUPED(DSV3_F16);
        default:        return DSV3_GROUPED(DSV3_F32);
    }
#undef DSV3_GROUPED
}

int dsv3_fp8_gemm_grouped(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                          const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                          void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                          const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                          int64_t num_tiles, void* stream) {
    return fp8_gemm_grouped_checked(a, a_s, a_rows, a_num_rows, b, b_s, b_group_stride, bs_group_stride, c, c_dtype,
                                    m, n, k, tile_group, tile_row0, tile_rows, num_tiles, stream, false);
}

int dsv3_fp8_gemm_grouped_pow2(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                               const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                               void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                               const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                               int64_t num_tiles, void* stream) {
    return fp8_gemm_grouped_checked(a, a_s, a_rows, a_num_rows, b, b_s, b_group_stride, bs_group_stride, c, c_dtype,
                                    m, n, k, tile_group, tile_row0, tile_rows, num_tiles, stream, true);
}

int dsv3_fp8_gemm_grouped_swiglu_fused(int64_t m, int64_t a_num_rows, int64_t inter, int64_t k) {
    return m > 0 && a_num_rows >= 0 && inter > 0 && k > 0 && k % 128 == 0 && m <= 0x7fffffff && 2 * inter <= 0x7fffffff &&
           k <= 0x7fffffff && grouped_swiglu_supported(m, a_num_rows, inter, k);
}

int dsv3_fp8_gemm_grouped_swiglu(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                                 const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                                 void* y, float* s, int64_t m, int64_t inter, int64_t k,
                                 const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                                 int64_t num_tiles, int block_size, int scale_fmt, void* stream) {
    if (scale_fmt != DSV3_SCALE_FMT_NONE && scale_fmt != DSV3_SCALE_FMT_UE8M0) return DSV3_ERR_BAD_DTYPE;
    if (block_size != 128) return DSV3_ERR_BAD_BLOCK;
    if (m < 0 || inter < 0 || k < 0 || a_num_rows < 0 || num_tiles < 0 || b_group_stride < 0 || bs_group_stride < 0)
        return DSV3_ERR_BAD_SHAPE;
    if (k % 128 != 0 || k == 0 || inter % 128 != 0) return DSV3_ERR_BAD_SHAPE;
    if (m == 0 || inter == 0 || num_tiles == 0) return DSV3_OK;
    if (!dsv3_fp8_gemm_grouped_swiglu_fused(m, a_num_rows, inter, k)) return DSV3_ERR_BAD_SHAPE;   // ask ..._fused first
    if (!a || !a_s || !b || !b_s || !y || !s || !tile_group || !tile_row0 || !tile_rows) return DSV3_ERR_NULL_POINTER;
    if (!aligned(a, 16) || !aligned(b, 16) || b_group_stride % 16 != 0 || !aligned(a_s, 4) || !aligned(b_s, 4) ||
        !aligned(y, 16) || !aligned(s, 4))
        return DSV3_ERR_MISALIGNED;
    return launch_grouped_swiglu(a, a_s, a_rows, b, b_s, y, s, m, inter, k, num_tiles, tile_group, tile_row0, tile_rows,
                                 b_group_stride, bs_group_stride, scale_fmt, (hipStream_t)stream);
}

int dsv3_swiglu_quant(const void* h, int h_dtype, void* y, float* s, int64_t rows, int64_t inter,
                      int block_size, int scale_fmt, void* stream) {
    if (h_dtype != DSV3_BF16) return DSV3_ERR_BAD_DTYPE;
    if (scale_fmt != DSV3_SCALE_FMT_NONE && scale_fmt != DSV3_SCALE_FMT_UE8M0) return DSV3_ERR_BAD_DTYPE;
    if (block_size != 128) return DSV3_ERR_BAD_BLOCK;
    if (rows < 0 || inter < 0 || inter % 128 != 0) return DSV3_ERR_BAD_SHAPE;
    if (rows == 0 || inter == 0) return DSV3_OK;
    if (!h || !y || !s) return DSV3_ERR_NULL_POINTER;
    if (!aligned(h, 16) || !aligned(y, 8) || !aligned(s, 4)) return DSV3_ERR_MISALIGNED;
    return launch_swiglu_quant(h, y, s, rows, inter, scale_fmt, (hipStream_t)stream);
}

int dsv3_moe_combine(const void* expert_out, int dtype, const int32_t* rows, const void* weights,
                     const void* shared, void* y, int64_t tokens, int topk, int64_t dim, void* stream) {
    if (dtype != DSV3_BF16) return DSV3_ERR_BAD_DTYPE;
    if (tokens < 0 || topk < 0 || dim < 0 || dim % 8 != 0 || tokens > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (tokens == 0 || dim == 0) return DSV3_OK;
    if (!y || (topk > 0 && (!expert_out || !rows || !weights))) return DSV3_ERR_NULL_POINTER;
    if (!aligned(expert_out, 16) || !aligned(shared, 16) || !aligned(y, 16)) return DSV3_ERR_MISALIGNED;
    return launch_moe_combine(expert_out, rows, weights, shared, y, tokens, topk, dim, (hipStream_t)stream);
}

int dsv3_gate_route(const void* logits, int dtype, const float* bias, void* weights, int64_t* indices,
                    int64_t tokens, int experts, int topk, int n_groups, int topk_groups, int score_func,
                    float route_scale, void* stream) {
    if (dtype != DSV3_BF16) return DSV3_ERR_BAD_DTYPE;
    if (score_func != DSV3_SCORE_SOFTMAX && score_func != DSV3_SCORE_SIGMOID) return DSV3_ERR_BAD_DTYPE;
    if (tokens < 0 || tokens > 0x7fffffff || experts < 1 || experts > 512 || topk < 1 || topk > 64 || topk > experts)
        return DSV3_ERR_BAD_SHAPE;
    if (n_groups < 1 || n_groups > 64 || experts % n_groups != 0 || topk_groups < 1 || topk_groups > n_groups ||
        (int64_t)topk_groups * (experts / n_groups) < topk)
        return DSV3_ERR_BAD_SHAPE;
    if (tokens == 0) return DSV3_OK;
    if (!logits || !weights || !indices) return DSV3_ERR_NULL_POINTER;
    if (!aligned(logits, 2) || !aligned(weights, 2) || !aligned(indices, 8) || !aligned(bias, 4)) return DSV3_ERR_MISALIGNED;
    return launch_gate_route(logits, bias, weights, indices, tokens, experts, topk, n_groups, topk_groups, score_func,
                             route_scale, (hipStream_t)stream);
}

int dsv3_wkv_b_absorb(const void* x, int64_t x_token_stride, int64_t x_head_stride,
                      const void* wkv_b, const float* wkv_b_scale, void* y, int dtype, int side,
                      int64_t tokens, int heads, int nope_dim, int v_dim, int64_t kv_rank, int block_size,
                      void* stream) {
    if (dtype != DSV3_BF16) return DSV3_ERR_BAD_DTYPE;
    if (block_size != 128) return DSV3_ERR_BAD_BLOCK;
    if (side != DSV3_ABSORB_Q && side != DSV3_ABSORB_V) return DSV3_ERR_BAD_SHAPE;
    if (tokens < 0 || heads < 0 || heads > 65535 || tokens > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
    if (!wkv_b_absorb_supported(side, nope_dim, v_dim, kv_rank)) return DSV3_ERR_BAD_SHAPE;
    const int64_t in_dim = side == DSV3_ABSORB_Q ? nope_dim : kv_rank;
    if (x_token_stride < 0 || x_head_stride < in_dim || x_token_stride % 8 != 0 || x_head_stride % 8 != 0)
        return DSV3_ERR_BAD_SHAPE;
    if (tokens == 0 || heads == 0) return DSV3_OK;
    if (!x || !wkv_b || !wkv_b_scale || !y) return DSV3_ERR_NULL_POINTER;
    if (!aligned(x, 16) || !aligned(wkv_b, 16) || !aligned(y, 16) || !aligned(wkv_b_scale, 4)) return DSV3_ERR_MISALIGNED;
    return launch_wkv_b_absorb(x, x_token_stride, x_head_stride, wkv_b, wkv_b_scale, y, side, tokens, heads,
                               nope_dim, v_dim, kv_rank, (hipStream_t)stream);
}

}  // extern "C"
