/* expf as the C library of the reference's hosts computes it, for host and device code.
 *
 * glibc 2.27 and later (the algorithm of ARM's optimized routines): the argument scaled by
 * 32 / ln 2 in double, the nearest integer k split off with the 1.5 * 2^52 shift, the remainder
 * by one fused multiply-add, 2^(k / 32) from a 32-entry table of doubles with k's upper bits added
 * into the exponent field, times a cubic in the remainder evaluated with three fused multiply-adds,
 * rounded to float once.  The fused steps are the ones the library's build for processors with FMA
 * makes (x86-64 with FMA, AArch64); every step is an IEEE double operation, so the result is that
 * library's bit for bit.  tests/check_expf.c compares this function with the host's expf (all 2^32
 * arguments with --all; the library's build without FMA differs on two of them by one ulp).
 * Compiled for the device under hipcc and for the host under a C compiler.
 * Table entry i holds the bits of 2^(i / 32) minus i << 47. */
#ifndef PF_EXPF_LIBM_H
#define PF_EXPF_LIBM_H
#include <stdint.h>

#ifdef __HIPCC__
#define PF_EXPF_FN __device__ static inline
#define PF_EXPF_TABLE __device__ static const
#else
#define PF_EXPF_FN static inline
#define PF_EXPF_TABLE static const
#endif

PF_EXPF_TABLE uint64_t pf_exp2_table[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

PF_EXPF_FN float pf_expf_libm(float x) {
#ifdef __clang__
#pragma clang fp contract(off)   /* only the four written fused steps; gcc: build with -ffp-contract=off */
#endif
    union { double d; uint64_t u; } bits;
    union { float f; uint32_t u; } inf;
    inf.u = 0x7f800000u;
    if (!(x <= 88.72283935546875f)) return x != x ? x : inf.f;   /* overflow beyond 0x1.62e42ep6 */
    if (x < -103.97207641601562f) return 0.0f;                    /* underflow below -0x1.9fe368p6 */
    const double scale = 0x1.71547652b82fep+0 * 32.0, shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0, c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0,
                 c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const double xd = (double)x;
    double kd = scale * xd;
    kd = kd + shift;
    bits.d = kd;
    const uint64_t ki = bits.u;
    kd = kd - shift;
    const double r = __builtin_fma(scale, xd, -kd);
    bits.u = pf_exp2_table[ki & 31u] + (ki << 47);
    const double s = bits.d;
    const double z = __builtin_fma(c0, r, c1);
    const double r2 = r * r;
    double y = __builtin_fma(c2, r, 1.0);
    y = __builtin_fma(z, r2, y);
    y = y * s;
    return (float)y;
}

/* The reference's sigmoid (src/qwen4_cpu_internal.h:103-106): both of its branches need expf(-|x|),
 * 1 / (1 + e) for x >= 0 and e / (1 + e) below. */
PF_EXPF_FN float pf_sigmoid_libm(float x) {
#ifdef __clang__
#pragma clang fp contract(off)
#endif
    const float e = pf_expf_libm(x < 0.0f ? x : -x);
    return (x >= 0.0f ? 1.0f : e) / (1.0f + e);
}
#endif
