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
 * Around them, each documented at its declaration: dsv3_linear_fp8 (the two calls of linear() as one launch for
 * few rows), dsv3_fp8_gemm_pow2 / dsv3_fp8_gemm_grouped_pow2 (power-of-two scales), dsv3_weight_quant (the inverse
 * of weight_dequant), the mixture-of-experts functions (dsv3_gate_route, dsv3_moe_route, dsv3_group_tiles,
 * dsv3_fp8_gemm_grouped, dsv3_fp8_gemm_grouped_swiglu, dsv3_swiglu_quant, dsv3_moe_combine) and
 * dsv3_wkv_b_absorb (attention).
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
    DSV3_ERR_LAUNCH = 7,        /* HIP reported an error at launch                         */
    DSV3_ERR_TOO_LARGE = 8      /* dsv3_fp8_gemm_static: scratch need exceeds the fixed array */
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

/* Which of the two wkv_b products of the absorbed attention dsv3_wkv_b_absorb computes. */
typedef enum dsv3_absorb_side {
    DSV3_ABSORB_Q = 0,   /* "bshd,hdc->bshc" with wkv_b[:, :nope]   (inference/model.py:483) */
    DSV3_ABSORB_V = 1    /* "bshc,hdc->bshd" with wkv_b[:, -v:]     (inference/model.py:495) */
} dsv3_absorb_side;

/* score_func of the router (inference/model.py:578-581). */
typedef enum dsv3_score_func {
    DSV3_SCORE_SOFTMAX = 0,
    DSV3_SCORE_SIGMOID = 1
} dsv3_score_func;

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
 * Any block_size >= 1 (32, 64, 128, 256 and 512 take the vectorised kernel, every other
 * size one wavefront per block).  x must be 16-byte aligned, y 8-byte, s 4-byte.
 * numel == 0 is a no-op.  The result is bit-identical to the IEEE evaluation of
 * the formula above.  Non-finite inputs follow that evaluation as torch's CPU operators
 * carry it out (amax propagates NaN), in both scale formats: a block that holds a NaN gets
 * s = NaN and NaN codes throughout, a block that holds an infinity (and no NaN) gets
 * s = inf, zeros for its finite elements and NaN codes for the infinite ones.  (Whether
 * the reference's tl.max propagates or drops a NaN depends on the Triton version; this
 * behaviour is pinned against the torch evaluation only.)  The quantisers fused into
 * dsv3_linear_fp8, dsv3_swiglu_quant and dsv3_weight_quant form their scales the same way.
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
 * Weight block-quantiser, the inverse of weight_dequant and the producer of the checkpoint format the reference
 * loads (README_WEIGHTS.md:60-92: `weight` e4m3 + `weight_scale_inv` binary32 per 128 x 128 block, a block that
 * is not aligned to 128 is zero-padded before its scale is calculated and the padding removed afterwards; scale
 * tensor shape inference/model.py:184-187).  The reference ships only the dequantising direction; the rule here is
 * the one its activation quantiser uses on 1 x 128 blocks (inference/kernel.py:23-35), applied to the square block:
 *     s[i,j] = max(amax(|w| over block i,j), 1e-4) / 448;   y = e4m3( w / s[i / 128, j / 128] )   (RNE)
 * With scale_fmt DSV3_SCALE_FMT_UE8M0 the scale is rounded up to a power of two before the division, as act_quant
 * does for activations (inference/kernel.py:29-31): the block-scale format of checkpoints made for
 * inference/configs/config_v3.1.json:22, and what dsv3_fp8_gemm_pow2 requires of its weight.
 * w: [m,n] of w_dtype, y: [m,n] fp8 bytes, s: [ceil(m/128), ceil(n/128)] binary32.  block_size must be 128.
 * Any m, n >= 0; n % 8 == 0 with 16-byte aligned w and 8-byte aligned y takes the vectorised kernel.
 */
int dsv3_weight_quant(const void* w, int w_dtype, void* y, float* s,
                      int64_t m, int64_t n, int block_size, int scale_fmt, void* stream);

/*
 * fp8_gemm (inference/kernel.py:145-172):
 *     c[i,j] = c_dtype( sum_kb ( sum_{t<128} a[i,128kb+t] * b[j,128kb+t] )
 *                                * a_s[i,kb] * b_s[j/128,kb] )
 * a: [m,k] fp8, a_s: [m,ceil(k/128)] binary32, b: [n,k] fp8 (the weight, out x in),
 * b_s: [ceil(n/128), ceil(k/128)] binary32, c: [m,n] of c_dtype.  Products and sums
 * are binary32; the order of additions differs from the reference's.
 * Any m, n >= 0.  a and b must be 16-byte aligned.  The kernels are written for k a multiple of 128, which is what
 * act_quant produces (inference/kernel.py:52); any other k runs a plain fallback kernel that masks the last,
 * partial block as the reference's kernel does (kernel.py:145, 158-159; m <= 65535 there, no workspace).
 * `workspace` must hold at least dsv3_fp8_gemm_workspace_bytes(m,n,k) bytes
 * (256-byte aligned) when that is non-zero; its contents on entry are ignored
 * and are undefined on return.  Calls sharing a workspace must be ordered on
 * one stream.
 */
int dsv3_fp8_gemm(const void* a, const float* a_s, const void* b, const float* b_s,
                  void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                  void* workspace, size_t workspace_bytes, void* stream);

/*
 * dsv3_fp8_gemm for scales that are all powers of two: what act_quant produces with scale_fmt "ue8m0"
 * (inference/kernel.py:29-31) and what checkpoints made for that format store as block scales
 * (inference/configs/config_v3.1.json:22).  The caller guarantees it for every element of a_s and b_s; it is not
 * checked.  For M > 64 the block scales then travel in the E8M0 scale operands of the gfx950 matrix instruction
 * and all K blocks accumulate inside the matrix core (the binary32 multiply-add per block and output element of
 * the general kernel disappears; the result differs from dsv3_fp8_gemm's only in the rounding of the sums).
 * Other shapes run the same kernels as dsv3_fp8_gemm.  Same arguments, workspace and errors.
 */
int dsv3_fp8_gemm_pow2(const void* a, const float* a_s, const void* b, const float* b_s,
                       void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                       void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of scratch dsv3_fp8_gemm needs for this problem (0 when none). */
size_t dsv3_fp8_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k);

/*
 * dsv3_fp8_gemm without a workspace argument and without any allocation.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  Same arithmetic, kernels, argument checks and results as dsv3_fp8_gemm
 * (bit for bit); the partial sums of K-sliced plans go to a fixed array of DSV3_STATIC_SCRATCH_BYTES inside the
 * library's device image (each GPU the library runs on holds its own copy until the process ends) instead of a
 * caller's buffer.  A problem whose dsv3_fp8_gemm_workspace_bytes(m,n,k) exceeds that size is refused with
 * DSV3_ERR_TOO_LARGE before anything is launched (every DeepSeek-V3 projection up to 4096 rows fits).
 * The first call on a device looks the array's address up (hipGetSymbolAddress; no allocation) -- make that call
 * outside a graph capture.  The array keeps the previous call's contents; the kernels overwrite what they read, so
 * nothing has to be cleared.  All calls on one GPU share the array: calls that overlap in time on one GPU (two
 * streams, two threads) race; order them on one stream.
 */
#define DSV3_STATIC_SCRATCH_BYTES (64u << 20)
size_t dsv3_fp8_gemm_static_max_bytes(void);
int dsv3_fp8_gemm_static(const void* a, const float* a_s, const void* b, const float* b_s,
                         void* c, int c_dtype, int64_t m, int64_t n, int64_t k, void* stream);

/*
 * ---- Mixture-of-experts layer on the same GEMM (inference/model.py:601-633 Expert, :669-693 MoE.forward) ----
 *
 * The reference walks its experts one by one: bincount(...).tolist() (a host sync, :683), then per expert
 * where / gather / 3 x (act_quant + fp8_gemm) / scatter-add (:684-689).  The functions below compute the same
 * values with the token lists kept on the device: rows of the activation matrix are grouped by expert
 * ("groups"), every group is multiplied by its own weight matrix in one launch, and the weighted outputs are
 * summed per token in ascending expert order, rounding to bf16 where the reference's tensor ops round.
 */

/* Height of a tile slot of dsv3_fp8_gemm_grouped (256 today); dsv3_group_tiles cuts groups into slots of at most
 * this many rows.  The kernel runs a slot of more than 128 rows as one 256-row tile and a smaller one as a 128-row
 * tile, so one table serves a few rows per group as well as hundreds. */
int dsv3_fp8_gemm_grouped_tile_rows(void);

/*
 * The FP8 branch of linear() for few rows, act_quant followed by fp8_gemm (inference/model.py:159-160), in one
 * launch: the weight-streaming kernel quantises the bf16 activations x [m,k] itself, with act_quant's arithmetic
 * (inference/kernel.py:23-35), so c equals dsv3_act_quant + dsv3_fp8_gemm bit for bit.  Implemented where
 * dsv3_linear_fp8_fused(m, n, k) returns non-zero (today: shapes that dsv3_fp8_gemm sends to its M <= 16 kernel with
 * m*k <= 131072 -- one and two rows everywhere, up to 16 rows on short K ranges or narrow weights); other shapes
 * return DSV3_ERR_BAD_SHAPE and the caller issues the two calls.  x_dtype must be DSV3_BF16, block_size 128; workspace as for dsv3_fp8_gemm.
 */
int dsv3_linear_fp8_fused(int64_t m, int64_t n, int64_t k);
int dsv3_linear_fp8(const void* x, int x_dtype, const void* b, const float* b_s, void* c, int c_dtype,
                    int64_t m, int64_t n, int64_t k, int block_size, int scale_fmt,
                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * Tile table for dsv3_fp8_gemm_grouped from per-group row counts (device int32 [groups]; the counts the
 * reference takes from bincount at inference/model.py:683).  Groups are laid out back to back in row order;
 * group g gets ceil(counts[g] / tile_rows) consecutive tile slots.  Writes three device int32 arrays of
 * max_tiles entries: the group of each slot (-1 for unused slots), its first row and its row count.
 * max_tiles >= total_rows / tile_rows + groups always suffices.
 */
int dsv3_group_tiles(const int32_t* counts, int groups, int max_tiles,
                     int32_t* tile_group, int32_t* tile_row0, int32_t* tile_rows, void* stream);

/*
 * Routing bookkeeping of one MoE forward, on the device (inference/model.py:683-689: bincount, the per-expert
 * torch.where token lists, and the order in which the loop over experts touches a token):
 *     indices [tokens, topk] int64 (the router's expert choices), weights [tokens, topk] (2-byte dtype)  ->
 *     scratch [3*experts] int32: counts per expert, first row per expert, (internal cursor);
 *     a_rows  [tokens*topk]    : token behind every row of the expert-sorted row list (groups back to back);
 *     rows    [tokens, topk]   : for every token, its rows in that list in ascending expert order;
 *     w_sorted[tokens, topk]   : the routing weights in the same order;
 *     tile_group/tile_row0/tile_rows [max_tiles]: the tile table of dsv3_group_tiles for these counts.
 * The order of rows inside an expert's group is unspecified (it does not affect any result).  topk <= 16.
 * shared_group != 0 appends one more group, index `experts`, that EVERY token selects with weight 1.0 as its last
 * entry (its rows are in token order): the shared expert of inference/model.py:690 run as one more group of the
 * grouped GEMMs; adding it last with weight 1 is the reference's `y + z`.  Then scratch has 3*(experts+1) entries,
 * a_rows tokens*(topk+1), and rows / w_sorted have topk+1 columns.
 */
int dsv3_moe_route(const int64_t* indices, const void* weights, int w_dtype, int64_t tokens, int topk, int experts,
                   int shared_group, int max_tiles, int32_t* scratch, int32_t* a_rows, int32_t* rows, void* w_sorted,
                   int32_t* tile_group, int32_t* tile_row0, int32_t* tile_rows, void* stream);

/*
 * Grouped fp8_gemm (inference/kernel.py:145-172 applied per expert as in inference/model.py:684-689):
 *     for every tile slot t with group g = tile_group[t] >= 0, rows r in [tile_row0[t], tile_row0[t]+tile_rows[t]):
 *         c[r, :] = fp8_gemm( a[src(r), :], a_s[src(r), :], b + g*b_group_stride, b_s + g*bs_group_stride )
 *     src(r) = a_rows ? a_rows[r] : r
 * a: [a_num_rows, k] fp8, a_s: [a_num_rows, k/128]; a_rows (optional, device int32 [m]) gathers token rows;
 * b: per-group weights [n, k] fp8, b_group_stride bytes apart; b_s: per-group scales [ceil(n/128), k/128],
 * bs_group_stride floats apart; c: [m, n] of c_dtype.  Rows of c not covered by a tile are left untouched.
 * k % 128 == 0, k >= 128; a_num_rows*k and n*k below 2^32.
 */
int dsv3_fp8_gemm_grouped(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                          const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                          void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                          const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                          int64_t num_tiles, void* stream);

/* dsv3_fp8_gemm_grouped for scales that are all powers of two (see dsv3_fp8_gemm_pow2: the caller's guarantee for
 * every element of a_s and b_s).  The tile kernel then passes the block scales to the matrix instruction; launches
 * of few rows take the same weight-streaming kernel as dsv3_fp8_gemm_grouped. */
int dsv3_fp8_gemm_grouped_pow2(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                               const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                               void* c, int c_dtype, int64_t m, int64_t n, int64_t k,
                               const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                               int64_t num_tiles, void* stream);

/*
 * The first grouped GEMM of a SwiGLU expert block with the activation and the re-quantisation in its epilogue
 * (inference/model.py:633: w2(silu(w1 x) * w3 x); the act_quant is that of w2's linear(), inference/model.py:159):
 *     h = dsv3_fp8_gemm_grouped(a, ..., b = [w1 ; w3] per group) as bf16;  (y, s) = dsv3_swiglu_quant(h)
 * in one launch, bit for bit: a column tile multiplies with the matching 128 rows of w1 and of w3, so that it
 * holds both factors of its 128 outputs -- one quantisation block -- and writes e4m3 bytes and scales instead of
 * 16-bit sums (a quarter of the bytes, and the launch in between is gone).
 * b: per group [2 * inter, k] (w1 over w3), b_s: per group [2 * inter / 128, k / 128]; y: [m, inter] e4m3,
 * s: [m, inter / 128]; the other arguments as dsv3_fp8_gemm_grouped.  block_size must be 128 and inter a multiple
 * of it.  Only the tile kernel has this epilogue: dsv3_fp8_gemm_grouped_swiglu_fused(m, a_num_rows, inter, k) says
 * whether a launch qualifies (more rows in all than the weight-streaming kernel takes); the entry point returns
 * DSV3_ERR_BAD_SHAPE otherwise and the caller issues the two separate calls.
 */
int dsv3_fp8_gemm_grouped_swiglu_fused(int64_t m, int64_t a_num_rows, int64_t inter, int64_t k);
int dsv3_fp8_gemm_grouped_swiglu(const void* a, const float* a_s, const int32_t* a_rows, int64_t a_num_rows,
                                 const void* b, const float* b_s, int64_t b_group_stride, int64_t bs_group_stride,
                                 void* y, float* s, int64_t m, int64_t inter, int64_t k,
                                 const int32_t* tile_group, const int32_t* tile_row0, const int32_t* tile_rows,
                                 int64_t num_tiles, int block_size, int scale_fmt, void* stream);

/*
 * silu(h1) * h3 followed by act_quant, in one pass (inference/model.py:633 feeding the act_quant of w2's
 * linear(), inference/model.py:159, inference/kernel.py:23-35):
 *     g = bf16( bf16( silu(h1) ) * h3 );  (y, s) = act_quant(g, 128, scale_fmt)
 * h: [rows, 2*inter] with h1 = h[:, :inter], h3 = h[:, inter:] (the two projections of one grouped GEMM);
 * y: [rows, inter] e4m3; s: [rows, inter/128].  h_dtype must be DSV3_BF16 and block_size 128.
 */
int dsv3_swiglu_quant(const void* h, int h_dtype, void* y, float* s, int64_t rows, int64_t inter,
                      int block_size, int scale_fmt, void* stream);

/*
 * Weighted scatter-add of the expert outputs plus the shared expert (inference/model.py:689-693):
 *     y[t] = 0;  for j < topk:  y[t] = bf16( y[t] + bf16( expert_out[rows[t,j]] * weights[t,j] ) );
 *     if shared:  y[t] = bf16( y[t] + shared[t] )
 * rows: device int32 [tokens, topk], listing each token's rows of expert_out in ascending expert order (the
 * order in which the reference's loop over experts adds them); weights: [tokens, topk]; all tensors of
 * `dtype`, which must be DSV3_BF16; dim % 8 == 0.
 */
int dsv3_moe_combine(const void* expert_out, int dtype, const int32_t* rows, const void* weights,
                     const void* shared, void* y, int64_t tokens, int topk, int64_t dim, void* stream);

/*
 * Expert selection of the router, everything after its linear layer (inference/model.py:577-598):
 *     s = sigmoid(logits) rounded to bf16, or softmax(logits) in binary32;   sel = s + bias (binary32, bias optional)
 *     n_groups > 1: a group scores the sum of its two largest sel (with bias) or its largest (without); experts
 *                   outside the topk_groups best groups are masked to -inf
 *     indices = the topk largest sel in descending order (ties: lower index);   w = s[indices]
 *     sigmoid: w = bf16(w / bf16(sum w));   weights = bf16(w * route_scale)
 * logits: [tokens, experts] of `dtype` (DSV3_BF16 only), the output of the router's linear layer; bias: fp32
 * [experts] or NULL; weights: bf16 [tokens, topk]; indices: int64 [tokens, topk].
 * 1 <= topk <= 64, topk <= experts <= 512, experts % n_groups == 0, n_groups <= 64,
 * topk <= topk_groups * (experts / n_groups).
 */
int dsv3_gate_route(const void* logits, int dtype, const float* bias, void* weights, int64_t* indices,
                    int64_t tokens, int experts, int topk, int n_groups, int topk_groups, int score_func,
                    float route_scale, void* stream);

/*
 * The two per-head products of the absorbed MLA attention with the fp8 weight wkv_b, dequantised in flight
 * instead of through a weight_dequant call per step (inference/model.py:481-483 and :495):
 *     W = bf16( f32(wkv_b) * scale[row/128, col/128] )        (what weight_dequant would write, kernel.py:83-86)
 *     side DSV3_ABSORB_Q:  y[t, h, c] = sum_{d < nope_dim} x[t, h, d] * W[h*(nope_dim+v_dim) + d, c]
 *     side DSV3_ABSORB_V:  y[t, h, d] = sum_{c < kv_rank}  x[t, h, c] * W[h*(nope_dim+v_dim) + nope_dim + d, c]
 * accumulated in binary32 and rounded once to `dtype` (DSV3_BF16 only).
 * x: bf16, element (t, h, j) at x[t*x_token_stride + h*x_head_stride + j] (strides in elements, multiples of 8;
 * this takes the q_nope view of q without a copy); wkv_b: [heads*(nope_dim+v_dim), kv_rank] e4m3, row-major;
 * wkv_b_scale: [ceil(rows/128), kv_rank/128]; y: contiguous [tokens, heads, kv_rank] (Q) or [tokens, heads, v_dim] (V).
 * block_size must be 128; kv_rank % 128 == 0, nope_dim and v_dim multiples of 32; side Q implements nope_dim
 * 64 and 128, side V kv_rank 128, 256 and 512 (DSV3_ERR_BAD_SHAPE otherwise).  x, wkv_b and y 16-byte aligned.
 */
int dsv3_wkv_b_absorb(const void* x, int64_t x_token_stride, int64_t x_head_stride,
                      const void* wkv_b, const float* wkv_b_scale, void* y, int dtype, int side,
                      int64_t tokens, int heads, int nope_dim, int v_dim, int64_t kv_rank, int block_size,
                      void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DSV3_FP8_H */
