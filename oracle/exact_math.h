/*
 * TEST INFRASTRUCTURE - CPU checker only.  Nothing in the shipped package may
 * include, link or call anything in this directory.
 *
 * Scalar arithmetic of the checker, written so that every operation is a
 * single correctly-rounded IEEE-754 binary32 operation (add, mul, div, sqrt,
 * fused multiply-add) or integer bit manipulation.  Compile with
 * -ffp-contract=off so that the only fused operations are the explicit fmaf()
 * calls.  The transcendental functions are short polynomial kernels (Cephes
 * single-precision coefficients), not libm: libm results vary between
 * implementations, while these are reproducible bit for bit on any IEEE
 * machine.  Accuracy is pinned against libm in the tests (<= 2 ulp on the
 * ranges the VM uses).
 *
 * The reference computes these steps with torch CPU kernels
 * (megakernels/demos/latency/python_vm.py:53-56 rsqrt, :161 silu, :320-323
 * softmax/exp/log2, :372 exp2); torch's results differ from these by rounding
 * only.
 */
#ifndef MK_ORACLE_EXACT_MATH_H
#define MK_ORACLE_EXACT_MATH_H

#include <math.h>
#include <stdint.h>
#include <string.h>

static inline uint32_t orc_f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float orc_bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* bfloat16 <-> float.  Round to nearest, ties to even; NaN stays NaN. */
static inline float orc_bf16_to_f32(uint16_t h) { return orc_bits_f32((uint32_t)h << 16); }
static inline uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = orc_f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
/* value of f after a round trip through bfloat16 */
static inline float orc_round_bf16(float f) { return orc_bf16_to_f32(orc_f32_to_bf16(f)); }

/* exp(r) for |r| <= 0.5 ln 2 (+ a little): 1 + r + r^2 P(r), Horner with fmaf */
static inline float orc_exp_poly(float r) {
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float r2 = r * r;
    float y = fmaf(p, r2, r);
    return y + 1.0f;
}

/* y * 2^n for n in [-126, 127] by building the power of two from bits */
static inline float orc_scale_pow2(float y, int n) {
    return y * orc_bits_f32((uint32_t)(n + 127) << 23);
}

/* e^x.  Results below the normal range are flushed to zero; x above 88 gives
 * +inf.  NaN in, NaN out. */
static inline float orc_expf(float x) {
    if (x != x) return x;
    if (x > 88.0f) return INFINITY;
    if (x < -86.0f) return 0.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    return orc_scale_pow2(orc_exp_poly(r), (int)n);
}

/* 2^x with the same flush / overflow convention */
static inline float orc_exp2f(float x) {
    if (x != x) return x;
    if (x > 127.0f) return INFINITY;
    if (x < -125.0f) return 0.0f;
    float n = rintf(x);
    float f = x - n; /* exact */
    return orc_scale_pow2(orc_exp_poly(f * 0.693147180559945f), (int)n);
}

/* log2(x) for finite normal x > 0; log2(0) = -inf */
static inline float orc_log2f(float x) {
    if (x != x || x < 0.0f) return NAN;
    if (x == 0.0f) return -INFINITY;
    if (x == INFINITY) return INFINITY;
    uint32_t u = orc_f32_bits(x);
    int e = (int)(u >> 23) - 126;                         /* x = m 2^e, m in [0.5, 1) */
    float m = orc_bits_f32((u & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106781186547524f) { e -= 1; m = (m + m) - 1.0f; } else { m = m - 1.0f; }
    float z = m * m;
    float p = 7.0376836292e-2f;
    p = fmaf(p, m, -1.1514610310e-1f);
    p = fmaf(p, m, 1.1676998740e-1f);
    p = fmaf(p, m, -1.2420140846e-1f);
    p = fmaf(p, m, 1.4249322787e-1f);
    p = fmaf(p, m, -1.6668057665e-1f);
    p = fmaf(p, m, 2.0000714765e-1f);
    p = fmaf(p, m, -2.4999993993e-1f);
    p = fmaf(p, m, 3.3333331174e-1f);
    float y = (p * m) * z;
    y = fmaf(-0.5f, z, y);
    float ln_m = m + y;                                   /* ln of the mantissa part */
    return fmaf(ln_m, 1.44269504088896341f, (float)e);
}

#endif
