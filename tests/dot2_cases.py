"""Operand generators for the two-element bf16 dot product (acc + a.lo*b.lo + a.hi*b.hi).

Every class aims at one clause of the written-out definition in oracle/exact_math.h (orc_dot2_bf16): which
operand sets the adder's last place, truncation of the smaller addends, cancellation, carries beyond the
adder's top bit, zeros and denormals, overflow and non-finite inputs.  Used by the GPU test that compares the
definition with the instruction and by the script that wrote tests/golden/dot2_vectors.npz.
"""
import numpy as np


def _bf(s, e, m):
    return (np.asarray(s).astype(np.uint32) << 15) | (np.asarray(e).astype(np.uint32) << 7) | np.asarray(m).astype(np.uint32)


def _f32(s, e, m):
    return (np.asarray(s).astype(np.uint32) << 31) | (np.asarray(e).astype(np.uint32) << 23) | np.asarray(m).astype(np.uint32)


def _rb(rng, n, e):
    return _bf(rng.integers(0, 2, n), e, rng.integers(0, 128, n))


def _round_bf16(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32)


def realistic(rng, n):
    """weights of a few hundredths, activations of order one, accumulator a partial sum of such products"""
    a0, a1 = _round_bf16(0.02 * rng.standard_normal(n)), _round_bf16(0.02 * rng.standard_normal(n))
    b0, b1 = _round_bf16(rng.standard_normal(n)), _round_bf16(rng.standard_normal(n))
    scale = rng.choice([0.0, 0.05, 1.0, 4.0, 30.0], n)
    acc = (0.02 * rng.standard_normal(n) * scale).astype(np.float32)
    return a0 | (a1 << 16), b0 | (b1 << 16), acc.view(np.uint32)


def one_product(rng, n):
    """second product zero (also zero times a huge partner), accumulator 45 binades either side of the product"""
    gap = rng.integers(-45, 46, n)
    ea = 127 + gap // 2
    a0, b0 = _rb(rng, n, ea), _rb(rng, n, 127 + gap - gap // 2)
    a1 = _rb(rng, n, rng.integers(1, 255, n))
    b1 = _bf(rng.integers(0, 2, n), np.zeros(n, int), np.zeros(n, int))
    acc = _f32(rng.integers(0, 2, n), np.full(n, 127), rng.integers(0, 1 << 23, n))
    swap = rng.integers(0, 2, n).astype(bool)
    return np.where(swap, a1 | (a0 << 16), a0 | (a1 << 16)), np.where(swap, b1 | (b0 << 16), b0 | (b1 << 16)), acc


def two_products(rng, n):
    """accumulator zero, second product up to 45 binades below the first"""
    gap = rng.integers(0, 46, n)
    a0, b0 = _rb(rng, n, np.full(n, 127)), _rb(rng, n, np.full(n, 127))
    a1, b1 = _rb(rng, n, 127 - gap // 2), _rb(rng, n, 127 - (gap - gap // 2))
    return a0 | (a1 << 16), b0 | (b1 << 16), _f32(rng.integers(0, 2, n), np.zeros(n, int), np.zeros(n, int))


def three_terms(rng, n):
    """independent gaps of up to 30 binades between each product and the accumulator"""
    g0, g1 = rng.integers(-30, 31, n), rng.integers(-30, 31, n)
    a0, b0 = _rb(rng, n, 127 + g0 // 2), _rb(rng, n, 127 + g0 - g0 // 2)
    a1, b1 = _rb(rng, n, 127 + g1 // 2), _rb(rng, n, 127 + g1 - g1 // 2)
    return a0 | (a1 << 16), b0 | (b1 << 16), _f32(rng.integers(0, 2, n), np.full(n, 127), rng.integers(0, 1 << 23, n))


def close_exponents(rng, n):
    """all three addends within two binades of each other: cancellation among them"""
    e = rng.integers(110, 140, n)
    a0, b0 = _rb(rng, n, e), _rb(rng, n, np.full(n, 127))
    a1, b1 = _rb(rng, n, e + rng.integers(-2, 3, n)), _rb(rng, n, np.full(n, 127))
    return a0 | (a1 << 16), b0 | (b1 << 16), _f32(rng.integers(0, 2, n), e + rng.integers(-2, 3, n), rng.integers(0, 1 << 23, n))


def cancelling_products(rng, n):
    """second product the negative of the first (or one bf16 step off), accumulator 40 binades either side"""
    e0, eb = rng.integers(100, 150, n), rng.integers(100, 150, n)
    a0, b0 = _rb(rng, n, e0), _rb(rng, n, eb)
    a1 = a0 ^ 0x8000
    b1 = np.where(rng.integers(0, 3, n) == 0, b0 ^ 1, b0)
    ec = np.clip(e0 + eb - 127 + rng.integers(-40, 41, n), 1, 254)
    return a0 | (a1 << 16), b0 | (b1 << 16), _f32(rng.integers(0, 2, n), ec, rng.integers(0, 1 << 23, n))


def carries(rng, n):
    """accumulator with leading ones and products just small enough to leave the last place to it: the sum
    reaches the bit above the adder's top"""
    ec, sc = rng.integers(60, 200, n), rng.integers(0, 2, n)
    k = rng.integers(2, 24, n)
    mant = ((1 << 23) - (1 << (23 - k))) | (rng.integers(0, 1 << 23, n) & ((1 << (23 - k)) - 1))
    acc = _f32(sc, ec, mant)
    e0 = ec - 7 - rng.integers(0, 9, n)
    ea0 = rng.integers(20, 120, n)
    eb0 = np.clip(e0 + 127 - ea0, 1, 254)
    e1 = e0 - rng.integers(0, 24, n)
    ea1 = rng.integers(20, 120, n)
    eb1 = np.clip(e1 + 127 - ea1, 1, 254)
    s0 = np.where(rng.integers(0, 5, n) == 0, 1 - sc, sc)
    s1 = np.where(rng.integers(0, 3, n) == 0, 1 - sc, sc)
    hi = lambda: np.where(rng.integers(0, 2, n) == 0, rng.integers(96, 128, n), rng.integers(0, 128, n))
    a0, b0 = _bf(s0, ea0, hi()), _bf(np.zeros(n, int), eb0, hi())
    a1, b1 = _bf(s1, ea1, hi()), _bf(np.zeros(n, int), eb1, hi())
    return a0 | (a1 << 16), b0 | (b1 << 16), acc


def near_power_of_two(rng, n):
    """accumulator at or just above a power of two (small exponents included), products mostly of the other
    sign and up to 33 binades below: the result lands one binade down, where one more bit of the small
    addends counts"""
    ec = np.where(rng.integers(0, 3, n) == 0, rng.integers(1, 40, n), rng.integers(40, 200, n))
    sc = rng.integers(0, 2, n)
    mant = np.where(rng.integers(0, 4, n) == 0, 0, rng.integers(0, 1 << 23, n) >> rng.integers(0, 24, n))
    acc = _f32(sc, ec, mant)
    e0 = ec - rng.integers(1, 34, n)
    ea0 = rng.integers(1, 120, n)
    eb0 = np.clip(e0 + 127 - ea0, 0, 254)
    e1 = e0 - rng.integers(0, 24, n)
    ea1 = rng.integers(1, 120, n)
    eb1 = np.clip(e1 + 127 - ea1, 0, 254)
    s0 = np.where(rng.integers(0, 5, n) == 0, sc, 1 - sc)
    s1 = np.where(rng.integers(0, 3, n) == 0, sc, 1 - sc)
    a0, b0 = _bf(s0, ea0, rng.integers(0, 128, n)), _bf(np.zeros(n, int), eb0, rng.integers(0, 128, n))
    a1, b1 = _bf(s1, ea1, rng.integers(0, 128, n)), _bf(np.zeros(n, int), eb1, rng.integers(0, 128, n))
    return a0 | (a1 << 16), b0 | (b1 << 16), acc


def tiny(rng, n):
    """denormal or zero accumulators (either sign), denormal bf16 operands, results in the denormal range"""
    e = lambda: rng.choice([0, 0, 1, 2, 30, 60, 64, 100, 126, 127], n)
    m = lambda: np.where(rng.integers(0, 4, n) == 0, 0, rng.integers(0, 128, n))
    a0, b0 = _bf(rng.integers(0, 2, n), e(), m()), _bf(rng.integers(0, 2, n), e(), m())
    a1, b1 = _bf(rng.integers(0, 2, n), e(), m()), _bf(rng.integers(0, 2, n), e(), m())
    acc = _f32(rng.integers(0, 2, n), rng.choice([0, 0, 1, 2, 20, 40], n), np.where(rng.integers(0, 3, n) == 0, 0, rng.integers(0, 1 << 23, n)))
    return a0 | (a1 << 16), b0 | (b1 << 16), acc


def any_bits(rng, n):
    """uniformly random bit patterns: infinities, NaNs, overflowing products included"""
    r = lambda: rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    return r(), r(), r()


def wide_finite(rng, n):
    """finite operands with exponents over the whole range: products beyond the fp32 range, huge cancellations"""
    e = lambda: rng.integers(0, 255, n)
    a0, b0, a1, b1 = _rb(rng, n, e()), _rb(rng, n, e()), _rb(rng, n, e()), _rb(rng, n, e())
    return a0 | (a1 << 16), b0 | (b1 << 16), _f32(rng.integers(0, 2, n), e(), rng.integers(0, 1 << 23, n))


CLASSES = [realistic, one_product, two_products, three_terms, close_exponents, cancelling_products, carries,
           near_power_of_two, tiny, any_bits, wide_finite]


def same_results(got, want):
    """bit-equal float32 arrays (given as uint32), any NaN matching any NaN"""
    g, w = np.asarray(got, dtype=np.uint32), np.asarray(want, dtype=np.uint32)
    nan = lambda u: (u & 0x7FFFFFFF) > 0x7F800000
    return (g == w) | (nan(g) & nan(w))
