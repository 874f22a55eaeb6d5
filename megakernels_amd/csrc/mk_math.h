// Scalar arithmetic of the megakernel's instruction epilogues.
//
// Every function is a fixed sequence of correctly rounded binary32 operations
// (add, mul, div, fused multiply-add) and integer bit manipulation, so the
// result is reproducible bit for bit on any IEEE-754 machine.  The kernel is
// built with -ffp-contract=off: only the explicit fmaf() calls fuse.  exp and
// log use Cephes' single-precision polynomial kernels (about 1 ulp) instead of
// the device's approximate v_exp_f32 / v_log_f32, whose results are not
// specified to the last bit.
//
// MK_HD lets the same file be compiled for the host by the test suite, which
// checks these functions against libm.
#pragma once

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define MK_HD __host__ __device__ __forceinline__
#else
#define MK_HD static inline
#endif

namespace mkm {

MK_HD uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
MK_HD float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// bf16 pair packed in one dword: element 0 in the low half
MK_HD float bf16_lo(uint32_t pair) { return bits_f32(pair << 16); }
MK_HD float bf16_hi(uint32_t pair) { return bits_f32(pair & 0xffff0000u); }

// float -> bf16 bits, round to nearest even, NaN stays NaN: the portable formula
MK_HD uint32_t f32_to_bf16_soft(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
#if defined(__HIP_DEVICE_COMPILE__)
// gfx950 converts in one instruction (v_cvt_pk_bf16_f32).  For every non-NaN input it returns the
// bits of the portable formula; the library's self test sweeps all 2^32 inputs to prove it.
MK_HD uint32_t f32_to_bf16(float f) { return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f); }
MK_HD uint32_t pack_bf16(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
#else
MK_HD uint32_t f32_to_bf16(float f) { return f32_to_bf16_soft(f); }
MK_HD uint32_t pack_bf16(float lo, float hi) { return f32_to_bf16(lo) | (f32_to_bf16(hi) << 16); }
#endif
MK_HD float round_bf16(float f) { return bits_f32(f32_to_bf16(f) << 16); }

// e^r for |r| <= ~0.35
MK_HD float exp_poly(float r) {
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

MK_HD float scale_pow2(float y, int n) { return y * bits_f32((uint32_t)(n + 127) << 23); }

// e^x; underflow is flushed to zero before the result would go subnormal
MK_HD float expf_exact(float x) {
    if (x != x) return x;
    if (x > 88.0f) return INFINITY;
    if (x < -86.0f) return 0.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    return scale_pow2(exp_poly(r), (int)n);
}

// 2^x
MK_HD float exp2f_exact(float x) {
    if (x != x) return x;
    if (x > 127.0f) return INFINITY;
    if (x < -125.0f) return 0.0f;
    float n = rintf(x);
    float f = x - n;
    return scale_pow2(exp_poly(f * 0.693147180559945f), (int)n);
}

// log2(x), x > 0 finite and normal
MK_HD float log2f_exact(float x) {
    if (x != x || x < 0.0f) return NAN;
    if (x == 0.0f) return -INFINITY;
    if (x == INFINITY) return INFINITY;
    uint32_t u = f32_bits(x);
    int e = (int)(u >> 23) - 126;
    float m = bits_f32((u & 0x007fffffu) | 0x3f000000u);  // [0.5, 1)
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
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
    float ln_m = m + y;
    return fmaf(ln_m, 1.44269504088896341f, (float)e);
}

// silu(g) = g / (1 + e^-g)
MK_HD float silu_exact(float g) { return g / (1.0f + expf_exact(-g)); }

}  // namespace mkm
