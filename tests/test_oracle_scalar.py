"""Pins the oracle's scalar arithmetic with independent exact mathematics
(Python big integers / Fractions), the examples worked out from the reference's
source text, and algebraic identities.  None of these tests retypes the
oracle's formula: each states what the number must be."""
import math
import random
from fractions import Fraction

import numpy as np
import pytest

import oracle_lib as O

I32_MIN, I32_MAX = -(1 << 31), (1 << 31) - 1


def wrap32(v):
    v &= 0xFFFFFFFF
    return v - (1 << 32) if v >= (1 << 31) else v


def trunc_div(a, b):
    """C '/' on integers: toward zero (exact, big ints)."""
    q = abs(a) // abs(b)
    return q if (a >= 0) == (b >= 0) else -q


def srdhm_by_c_rules(a, b):
    ab = a * b
    nudge = (1 << 30) if ab >= 0 else 1 - (1 << 30)
    return wrap32(trunc_div(ab + nudge, 1 << 31))


def nearest_ties_up(fr):
    """nearest integer to a Fraction, ties toward +inf"""
    return math.floor(fr + Fraction(1, 2))


def nearest_ties_away(fr):
    s = -1 if fr < 0 else 1
    return s * math.floor(abs(fr) + Fraction(1, 2))


def structured_i32():
    vals = {0, 1, -1, 2, -2, 3, -3, I32_MIN, I32_MAX, I32_MIN + 1, I32_MAX - 1}
    for k in range(1, 31):
        for d in (-1, 0, 1):
            vals.add((1 << k) + d)
            vals.add(-(1 << k) + d)
    return sorted(vals)


def test_srdhm_worked_examples():
    # ties go toward +inf: -1 * 2^30 / 2^31 = -0.5 -> 0 ; -3 -> -1.5 -> -1 ; 1 -> 0.5 -> 1
    assert O.lib.orc_srdhm(-1, 1 << 30) == 0
    assert O.lib.orc_srdhm(-3, 1 << 30) == -1
    assert O.lib.orc_srdhm(1, 1 << 30) == 1
    assert O.lib.orc_srdhm(3, 1 << 30) == 2


def test_srdhm_is_round_to_nearest_ties_up_on_structured_grid():
    vs = structured_i32()
    for a in vs:
        for b in vs:
            exact = nearest_ties_up(Fraction(a * b, 1 << 31))
            assert srdhm_by_c_rules(a, b) == wrap32(exact)
            assert O.lib.orc_srdhm(a, b) == wrap32(exact), (a, b)


def test_srdhm_random():
    rng = random.Random(1234)
    for _ in range(20000):
        a = rng.randint(I32_MIN, I32_MAX)
        b = rng.randint(1 << 30, I32_MAX)
        assert O.lib.orc_srdhm(a, b) == nearest_ties_up(Fraction(a * b, 1 << 31))


def test_srdhm_identity_multiplier_2_30_is_half_round_up():
    # multiplier 2^30 halves: floor((v+1)/2)
    for v in structured_i32():
        assert O.lib.orc_srdhm(v, 1 << 30) == (v + 1) // 2


def test_rdbp_worked_examples():
    assert O.lib.orc_rdbp(-1, 1) == -1
    assert O.lib.orc_rdbp(1, 1) == 1
    assert O.lib.orc_rdbp(-3, 1) == -2
    assert O.lib.orc_rdbp(0, 5) == 0
    assert O.lib.orc_rdbp(12345, 0) == 12345


def test_rdbp_is_round_to_nearest_ties_away_everywhere():
    vs = structured_i32()
    for e in range(1, 32):
        for x in vs:
            assert O.lib.orc_rdbp(x, e) == nearest_ties_away(Fraction(x, 1 << e)), (x, e)
        # every tie and its neighbours around a few multiples
        half = 1 << (e - 1)
        for mult in (-5, -3, -1, 1, 3, 5):
            for d in (-1, 0, 1):
                x = mult * half + d
                if I32_MIN <= x <= I32_MAX:
                    assert O.lib.orc_rdbp(x, e) == nearest_ties_away(Fraction(x, 1 << e)), (x, e)


def test_rdbp_random():
    rng = random.Random(99)
    for _ in range(20000):
        x = rng.randint(I32_MIN, I32_MAX)
        e = rng.randint(1, 31)
        assert O.lib.orc_rdbp(x, e) == nearest_ties_away(Fraction(x, 1 << e))


def test_saturate_int8_half_up_and_clamp():
    cases = [(0.5, 1), (-0.5, 0), (1.5, 2), (-1.5, -1), (2.5, 3), (-2.5, -2), (126.5, 127),
             (127.4, 127), (127.5, 127), (1e9, 127), (-128.5, -128), (-128.51, -128),
             (-1e9, -128), (0.49999997, 0), (-0.50000006, -1), (3e38, 127), (-3e38, -128)]
    for f, want in cases:
        f32 = float(np.float32(f))
        exact = max(-128, min(127, math.floor(Fraction(f32) + Fraction(1, 2))))
        assert exact == want, (f, exact, want)
        assert O.lib.orc_saturate_int8(f32) == want, f


def test_saturate_int8_random_floats():
    rng = np.random.default_rng(5)
    xs = np.concatenate([rng.uniform(-300, 300, 5000), rng.integers(-300, 300, 2000) + 0.5,
                         rng.uniform(-1, 1, 2000) * 1e-3]).astype(np.float32)
    for f in xs:
        f = float(f)
        exact = max(-128, min(127, math.floor(Fraction(f) + Fraction(1, 2))))
        assert O.lib.orc_saturate_int8(f) == exact


def test_apply_rshift_matches_integer_half_up_shift():
    # v / 2^r is exact in float for |v| < 2^24, so the result is floor((v + 2^(r-1)) / 2^r)
    rng = random.Random(3)
    for _ in range(20000):
        v = rng.randint(-(1 << 23), 1 << 23)
        r = rng.randint(0, 20)
        exact = max(-128, min(127, math.floor(Fraction(v, 1 << r) + Fraction(1, 2))))
        assert O.lib.orc_apply_rshift_sat8(float(v), r) == exact


def test_qdm_int_is_two_roundings_then_clamp():
    rng = random.Random(7)
    for _ in range(20000):
        v = rng.randint(-(1 << 26), 1 << 26)
        m = rng.randint(1 << 30, I32_MAX)
        r = rng.randint(0, 31)
        s1 = nearest_ties_up(Fraction(v * m, 1 << 31))
        s2 = nearest_ties_away(Fraction(s1, 1 << r)) if r else s1
        want = max(-128, min(127, s2))
        assert O.lib.orc_apply_mult_rshift_sat8_i(v, r, m, 1) == want
        assert O.lib.orc_apply_mult_rshift_sat8_f(float(np.float32(v)), r, m, 1) == \
            O.lib.orc_apply_mult_rshift_sat8_i(int(np.float32(v)), r, m, 1)


def test_qdm_differs_from_single_rounding_somewhere():
    # the two-step rule is not a single round-half-up shift by 31+r; make sure the
    # oracle implements the former (a dropped rounding step would pass neither)
    rng = random.Random(11)
    diff = 0
    for _ in range(50000):
        v = rng.randint(-(1 << 20), 1 << 20)
        m = rng.randint(1 << 30, I32_MAX)
        r = rng.randint(8, 12)
        single = max(-128, min(127, math.floor(Fraction(v * m, 1 << (31 + r)) + Fraction(1, 2))))
        if O.lib.orc_apply_mult_rshift_sat8_i(v, r, m, 1) != single:
            diff += 1
    assert diff > 0


def test_non_qdm_float_overload_uses_float32_product():
    # exact while v*m < 2^24 ...
    rng = random.Random(13)
    for _ in range(10000):
        v = rng.randint(-6500, 6500)
        m = rng.randint(0, 255)
        r = rng.randint(0, 15)
        exact = max(-128, min(127, math.floor(Fraction(v * m, 1 << r) + Fraction(1, 2))))
        assert O.lib.orc_apply_mult_rshift_sat8_f(float(v), r, m, 0) == exact
    # ... and rounded to float32 beyond (16777217 is not a float32)
    v, m, r = 16777217.0, 3, 20
    prod = np.float32(np.float32(v)) * np.float32(m)
    exact = max(-128, min(127, math.floor(Fraction(float(prod)) / (1 << r) + Fraction(1, 2))))
    assert O.lib.orc_apply_mult_rshift_sat8_f(v, r, m, 0) == exact


def test_float_stored_multiplier_conversion():
    # multiples of 128 in [2^30, 2^31) survive the float32 round trip unchanged;
    # others move to the nearest float32; 2^31 - 1 rounds up to 2^31 -> INT_MIN as int32
    assert O.lib.orc_f2u32(float(np.float32((1 << 30) + 128))) == (1 << 30) + 128
    assert O.lib.orc_f2u32(float(np.float32((1 << 30) + 1))) == (1 << 30)
    u = O.lib.orc_f2u32(float(np.float32(I32_MAX)))
    assert u == 1 << 31 and wrap32(u) == I32_MIN
    assert O.lib.orc_f2u32(-1.0) == 0xFFFFFFFF  # x86-64 gcc wrap of a negative float
    assert O.lib.orc_f2u32(17.9) == 17
