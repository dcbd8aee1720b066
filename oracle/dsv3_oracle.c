/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by or called from the
 * shipped library.  Only tests/, the smoke check and the bench's cpu_baseline
 * leg may use this file.
 *
 * Plain-C restatement of the arithmetic of DeepSeek-V3's block-scaled FP8 path
 * (reference: inference/kernel.py).  Every conversion is written out with
 * integer bit manipulation so that it is independent of any library's float8 /
 * bfloat16 casts; the torch-CPU oracle (oracle/oracle.py) is pinned against it.
 *
 *   e4m3fn  = OCP FP8 E4M3: 1 sign, 4 exponent (bias 7), 3 mantissa bits,
 *             no infinities, S.1111.111 is NaN, largest finite 448.
 *   bf16    = upper 16 bits of an IEEE binary32, round-to-nearest-even.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bf16 bits -> binary32 (exact widening; kernel.py:25 `.to(tl.float32)`). */
float oracle_bf16_to_f32(uint16_t h) { return u32_as_f32((uint32_t)h << 16); }

/* binary32 -> bf16 bits, round-to-nearest-even; NaN stays a quiet NaN. */
uint16_t oracle_f32_to_bf16(float f) {
    uint32_t u = f32_as_u32(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* e4m3fn byte -> binary32 (exact). */
float oracle_e4m3_to_f32(uint8_t b) {
    uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    uint32_t e = (b >> 3) & 0xfu, m = b & 0x7u;
    if (e == 0xfu && m == 0x7u) return u32_as_f32(sign | 0x7fc00000u);
    float mag;
    if (e == 0) mag = ldexpf((float)m, -9);               /* subnormal: m * 2^-6 / 8 */
    else        mag = ldexpf((float)(8u + m), (int)e - 10); /* (1+m/8) * 2^(e-7)      */
    return sign ? -mag : mag;
}

/*
 * binary32 -> e4m3fn byte, round-to-nearest-even on the exact value
 * (kernel.py:33 `y.to(float8_e4m3fn)`).  Values that round above 448 (|v| >=
 * 464) have no finite encoding and give NaN (0x7f), as does NaN; the sign of
 * zero and of values that underflow to zero is kept.
 */
uint8_t oracle_f32_to_e4m3(float f) {
    uint32_t u = f32_as_u32(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);     /* NaN */
    if (a >= 0x43e80000u) return (uint8_t)(sign | 0x7fu);    /* >= 464: overflow (also inf) */
    int e = (int)(a >> 23) - 127;                            /* unbiased exponent */
    uint32_t man = (a & 0x7fffffu) | 0x800000u;              /* 24-bit significand */
    if ((a >> 23) == 0) { return sign; }                     /* f32 subnormal: far below 2^-10 */
    /* number of low significand bits to drop: 20 for normals, more for e4m3 subnormals */
    int drop = 20;
    if (e < -6) drop += (-6 - e);
    if (drop > 25) return sign;                              /* < 2^-11: rounds to zero */
    uint32_t keep = man >> drop;
    uint32_t rem = man & ((1u << drop) - 1u);
    uint32_t half = 1u << (drop - 1);
    if (rem > half || (rem == half && (keep & 1u))) keep += 1u;
    uint32_t out;
    if (e < -6) {
        out = keep;                /* subnormal field (keep==8 carries into the first normal) */
    } else {
        /* keep is in [8,16]; 16 means carry into the next exponent */
        uint32_t eb = (uint32_t)(e + 7);
        if (keep == 16u) { keep = 8u; eb += 1u; }
        out = (eb << 3) | (keep & 7u);
    }
    return (uint8_t)(sign | (uint8_t)out);
}

/* scale_fmt == "ue8m0": s -> 2^ceil(log2 s) (kernel.py:29-31), on the bits of a
 * positive normal binary32: a power of two is kept, anything else moves to the
 * next power of two. */
float oracle_ue8m0_round_up(float s) {
    uint32_t u = f32_as_u32(s);
    uint32_t e = u >> 23, m = u & 0x7fffffu;
    if (m) e += 1u;
    return u32_as_f32(e << 23);
}

/*
 * act_quant (kernel.py:23-35): for each run of `block` contiguous elements
 *   amax = max|x|; amax = max(amax, 1e-4f); s = amax / 448.f;
 *   [ue8m0: s = 2^ceil(log2 s)];  y = e4m3(x / s).
 * x: bf16 bits [rows*k]; y: bytes [rows*k]; s: [rows*k/block].
 */
void oracle_act_quant(const uint16_t* x, uint8_t* y, float* s,
                      int64_t numel, int block, int ue8m0) {
    for (int64_t b0 = 0; b0 < numel; b0 += block) {
        float amax = 0.f;
        for (int j = 0; j < block; ++j) {
            float v = fabsf(oracle_bf16_to_f32(x[b0 + j]));
            if (v > amax) amax = v;
        }
        if (amax < 1e-4f) amax = 1e-4f;
        volatile float sc = amax / 448.f;
        float scale = sc;
        if (ue8m0) scale = oracle_ue8m0_round_up(scale);
        s[b0 / block] = scale;
        for (int j = 0; j < block; ++j) {
            volatile float q = oracle_bf16_to_f32(x[b0 + j]) / scale;
            y[b0 + j] = oracle_f32_to_e4m3(q);
        }
    }
}

/*
 * weight_dequant (kernel.py:76-86): y[i,j] = bf16( f32(x[i,j]) * s[i/block, j/block] ),
 * scale row stride ceil(n/block).
 */
void oracle_weight_dequant(const uint8_t* x, const float* s, uint16_t* y,
                           int64_t m, int64_t n, int block) {
    int64_t sn = (n + block - 1) / block;
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            volatile float p = oracle_e4m3_to_f32(x[i * n + j]) * s[(i / block) * sn + j / block];
            y[i * n + j] = oracle_f32_to_bf16(p);
        }
}

/*
 * fp8_gemm (kernel.py:145-172):
 *   c[m,n] = sum_kb ( sum_j a[m,128kb+j] * b[n,128kb+j] ) * a_s[m,kb] * b_s[n/128,kb]
 * The inner dot product is evaluated exactly (every e4m3 product is exact in
 * binary32 and a double holds the sum of 128 of them without rounding); the
 * per-block result is rounded to binary32 once, scaled in binary32 in the
 * reference's order (dot*a_s)*b_s and accumulated in binary32.
 * a: [m,k] bytes, b: [n,k] bytes, a_s: [m,ceil(k/128)], b_s: [ceil(n/128), ceil(k/128)],
 * c32: [m,n] binary32, c16: [m,n] bf16 bits (either may be NULL).
 */
void oracle_fp8_gemm(const uint8_t* a, const float* a_s, const uint8_t* b, const float* b_s,
                     float* c32, uint16_t* c16, int64_t m, int64_t n, int64_t k) {
    float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3_to_f32((uint8_t)i);
    int64_t kb_n = (k + 127) / 128;           /* a last block of fewer than 128 values is masked (kernel.py:145, 158-159) */
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            float acc = 0.f;
            for (int64_t kb = 0; kb < kb_n; ++kb) {
                double dot = 0.0;
                const uint8_t* ap = a + i * k + kb * 128;
                const uint8_t* bp = b + j * k + kb * 128;
                const int len = (int)(k - kb * 128 < 128 ? k - kb * 128 : 128);
                for (int t = 0; t < len; ++t) dot += (double)lut[ap[t]] * (double)lut[bp[t]];
                volatile float d = (float)dot;
                volatile float d1 = d * a_s[i * kb_n + kb];
                volatile float d2 = d1 * b_s[(j / 128) * kb_n + kb];
                acc += d2;
            }
            if (c32) c32[i * n + j] = acc;
            if (c16) c16[i * n + j] = oracle_f32_to_bf16(acc);
        }
}
