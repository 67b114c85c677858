"""Pins for oracle/kernels_ref.c (CPU only): what the mathematics fixes."""

from fractions import Fraction

import numpy as np

from oracle import kernels_oracle as ko


def test_triad_is_one_rounding_of_the_exact_value():
    rng = np.random.default_rng(0)
    b = (rng.random(257, dtype=np.float32) * 2 - 1)
    c = (rng.random(257, dtype=np.float32) * 2 - 1)
    s = np.float32(1.7)
    got = ko.triad(b, c, float(s))
    for i in range(0, 257, 7):
        exact = Fraction(float(b[i])) + Fraction(float(s)) * Fraction(float(c[i]))
        # the correctly rounded fp32 of the exact rational value
        want = np.float32(float(exact))  # float(Fraction) rounds to nearest double;
        # double -> float could double-round, so check via neighbours instead
        lo, hi = np.nextafter(got[i], np.float32(-np.inf)), np.nextafter(got[i], np.float32(np.inf))
        err = abs(Fraction(float(got[i])) - exact)
        assert err <= abs(Fraction(float(lo)) - exact)
        assert err <= abs(Fraction(float(hi)) - exact)
        assert abs(float(want) - float(got[i])) <= abs(float(hi) - float(lo))


def test_triad_differs_from_two_roundings_somewhere():
    # a*b+c with a separate multiply rounds twice; FMA must not.  Hand case:
    # s = 1+2^-12, c = 1+2^-12, b = -(1+2^-11): exact = 2^-24, product rounds to 1+2^-11.
    s = np.float32(1 + 2.0 ** -12)
    c = np.array([1 + 2.0 ** -12], dtype=np.float32)
    b = np.array([-(1 + 2.0 ** -11)], dtype=np.float32)
    assert ko.triad(b, c, float(s))[0] == np.float32(2.0 ** -24)
    assert np.float32(s * c[0]) + b[0] == np.float32(0.0)


def test_triad_special_cases():
    b = np.array([0.0, -0.0, np.inf, 1.0, np.nan], dtype=np.float32)
    c = np.array([0.0, 0.0, 1.0, np.inf, 1.0], dtype=np.float32)
    got = ko.triad(b, c, 2.0)
    assert got[0] == 0 and got[2] == np.inf and got[3] == np.inf and np.isnan(got[4])
    assert ko.triad(np.empty(0, np.float32), np.empty(0, np.float32), 1.0).size == 0


def test_bf16_rounding_is_nearest_even():
    cases = {1.0: 0x3f80, 1.00390625: 0x3f80,     # 1 + 2^-8: tie -> even (down)
             1.01171875: 0x3f82,                   # 1 + 3*2^-8: tie -> even (up)
             1.0078125: 0x3f81, -2.5: 0xc020, 0.0: 0x0000}
    for value, bits in cases.items():
        assert ko.lib().oracle_f32_to_bf16(value) == bits
        assert ko.f32_to_bf16_bits(np.array([value]))[0] == bits
    assert ko.f32_to_bf16_bits(np.array([np.nan]))[0] & 0x7fc0 == 0x7fc0
    x = np.random.default_rng(1).standard_normal(1000).astype(np.float32)
    assert np.array_equal(ko.f32_to_bf16_bits(x),
                          np.array([ko.lib().oracle_f32_to_bf16(float(v)) for v in x], np.uint16))


def test_gemm_matches_exact_integer_products():
    # small integers are exact in bf16, so the product is an exact integer matrix
    rng = np.random.default_rng(2)
    a = rng.integers(-8, 9, (5, 64)).astype(np.float32)
    b = rng.integers(-8, 9, (7, 64)).astype(np.float32)
    got = ko.gemm_bf16_nt(ko.f32_to_bf16_bits(a), ko.f32_to_bf16_bits(b))
    assert np.array_equal(got, (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.float64))
    # transposed operand would fail this (A B^T != A^T B); row windows agree
    part = ko.gemm_bf16_nt(ko.f32_to_bf16_bits(a), ko.f32_to_bf16_bits(b), 2, 4)
    assert np.array_equal(part, got[2:4])
