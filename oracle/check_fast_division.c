/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * Enumerates the claim the act_quant kernel's quotient rests on: for bf16 x and
 * a scale s = max(amax,1e-4)/448 (optionally rounded up to a power of two) with
 * |x| <= amax,
 *      r = RN(1/s);  q0 = x*r;  e = fma(-q0, s, x);  q = copysign(fma(e, r, q0), x)
 * equals the IEEE quotient RN(x/s) whenever |x/s| >= 2^-12, and always encodes
 * to the same e4m3 byte.
 *
 *   check_fast_division [stride]   amax walks every stride-th positive finite bf16
 *                                  (stride 1 = exhaustive: 2^31 cases, ~10 s on 8 cores)
 * Exit status 0 and "mismatches=0" on success.
 */
#include <stdio.h>
#include <stdlib.h>
#include "dsv3_oracle.c"

int main(int argc, char** argv) {
    int stride = argc > 1 ? atoi(argv[1]) : 1;
    if (stride < 1) stride = 1;
    long bad_q = 0, bad_byte = 0, total = 0;
#pragma omp parallel for schedule(dynamic, 16) reduction(+ : bad_q, bad_byte, total)
    for (int ab = 1; ab < 0x7f80; ab += stride) {
        const float amax = oracle_bf16_to_f32((uint16_t)ab);
        const float am = amax < 1e-4f ? 1e-4f : amax;
        volatile float s0 = am / 448.f;
        for (int ue = 0; ue < 2; ++ue) {
            const float s = ue ? oracle_ue8m0_round_up(s0) : s0;
            volatile float rv = 1.0f / s;
            const float r = rv;
            for (int xb = 0; xb < 0x10000; ++xb) {
                if ((xb & 0x7f80) == 0x7f80) continue;
                const float x = oracle_bf16_to_f32((uint16_t)xb);
                if (fabsf(x) > amax) continue;
                volatile float qt = x / s;
                const float q0 = x * r;
                const float e = fmaf(-q0, s, x);
                const float q = copysignf(fmaf(e, r, q0), x);
                const float qtv = qt;
                ++total;
                if (f32_as_u32(q) != f32_as_u32(qtv) && fabsf(qtv) >= 0x1p-12f) ++bad_q;
                if (oracle_f32_to_e4m3(q) != oracle_f32_to_e4m3(qtv)) ++bad_byte;
            }
        }
    }
    printf("cases=%ld quotient_mismatches=%ld byte_mismatches=%ld mismatches=%ld\n",
           total, bad_q, bad_byte, bad_q + bad_byte);
    return (bad_q + bad_byte) ? 1 : 0;
}
