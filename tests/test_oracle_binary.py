"""Pins the oracle's two-input elementwise ops (max / min / mul, broadcast add / sub / mul)
against exact rational arithmetic and numpy's own broadcasting: the expected values are
computed from what the operation must be, not from the oracle's formula."""
import math
from fractions import Fraction

import numpy as np
import pytest

import oracle_lib as O
from test_oracle_scalar import nearest_ties_away, nearest_ties_up, srdhm_by_c_rules


def sat8(v):
    return max(-128, min(127, v))


def expect_linear(op, a, b, m0, m1, r, relu):
    """sat8(floor(relu?(op(a*m0, b*m1)) / 2^r + 1/2)) in exact arithmetic, elementwise"""
    a, b = np.broadcast_arrays(a.astype(np.int64) * m0, b.astype(np.int64) * m1)
    v = {O.BIN_ADD: a + b, O.BIN_SUB: a - b, O.BIN_MAX: np.maximum(a, b),
         O.BIN_MIN: np.minimum(a, b)}[op]
    if relu:
        v = np.maximum(v, 0)
    out = np.empty(v.shape, np.int8)
    for idx, x in np.ndenumerate(v):
        out[idx] = sat8(nearest_ties_up(Fraction(int(x), 1 << r)))
    return out


def expect_mul(a, b, mult, r, relu):
    a, b = np.broadcast_arrays(a.astype(np.int64), b.astype(np.int64))
    v = a * b
    if relu:
        v = np.maximum(v, 0)
    out = np.empty(v.shape, np.int8)
    for idx, x in np.ndenumerate(v):
        h = srdhm_by_c_rules(int(x), mult)
        out[idx] = sat8(nearest_ties_away(Fraction(h, 1 << r)) if r else h)
    return out


SHAPES = [((2, 5, 3, 4), (2, 5, 3, 4)),        # eltwise
          ((2, 5, 3, 4), (1, 5, 1, 1)),        # per-channel operand
          ((2, 5, 3, 4), (2, 1, 3, 4)),        # per-pixel operand
          ((1, 1, 3, 1), (2, 5, 1, 4)),        # both broadcast
          ((2, 5, 3, 4), (1, 1, 1, 1))]        # scalar


@pytest.mark.parametrize("op", [O.BIN_ADD, O.BIN_SUB, O.BIN_MAX, O.BIN_MIN])
@pytest.mark.parametrize("shapes", SHAPES)
@pytest.mark.parametrize("relu", [False, True])
def test_linear_binary_ops_match_exact_arithmetic(op, shapes, relu):
    rng = np.random.default_rng(op * 7 + len(shapes[1]) + relu)
    a = rng.integers(-128, 128, shapes[0]).astype(np.int8)
    b = rng.integers(-128, 128, shapes[1]).astype(np.int8)
    for m0, m1, r in [(1, 1, 0), (3, -2, 1), (127, 127, 7), (-128, 77, 8), (90, 45, 30)]:
        got = O.binary_i8(op, a, b, [m0, m1], r, relu)
        assert np.array_equal(got, expect_linear(op, a, b, m0, m1, r, relu)), (m0, m1, r)


def test_linear_ops_extremes_and_ties():
    a = np.array([-128, -128, 127, 127, 1, -1, 3, -3, 0], np.int8).reshape(1, 9, 1, 1)
    b = np.array([-128, 127, -128, 127, 0, 0, 0, 0, 0], np.int8).reshape(1, 9, 1, 1)
    # ties: 1/2 -> 1, -1/2 -> 0 (round half up), 3/2 -> 2, -3/2 -> -1
    got = O.binary_i8(O.BIN_ADD, a, b, [1, 1], 1)
    assert got.ravel().tolist() == [-128, 0, 0, 127, 1, 0, 2, -1, 0]
    got = O.binary_i8(O.BIN_ADD, a, b, [127, 127], 0)      # |sum| up to 32512: saturates
    assert got.ravel().tolist()[:4] == [-128, -127, -127, 127]   # -32512, -127, -127, 32258
    # the multiplier is converted to int8 before use: 200.0 -> (int8)200 = -56
    got = O.binary_i8(O.BIN_MAX, a, b, [200.0, 1.0], 0)
    want = expect_linear(O.BIN_MAX, a, b, -56, 1, 0, False)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shapes", SHAPES)
@pytest.mark.parametrize("relu", [False, True])
def test_mul_matches_exact_two_step_rounding(shapes, relu):
    rng = np.random.default_rng(len(shapes[1]) + relu)
    a = rng.integers(-128, 128, shapes[0]).astype(np.int8)
    b = rng.integers(-128, 128, shapes[1]).astype(np.int8)
    for mult, r in [(1 << 30, 7), (1518500250, 6), ((1 << 31) - 128, 14), (1 << 30, 0), (12345 * 128, 1)]:
        got = O.binary_i8(O.BIN_MUL, a, b, [float(mult)], r, relu)
        assert np.array_equal(got, expect_mul(a, b, mult, r, relu)), (mult, r)


def test_mul_without_requant_is_refused():
    a = np.ones((1, 1, 1, 1), np.int8)
    with pytest.raises(ValueError):
        O.binary_i8(O.BIN_MUL, a, a, [0.0], 0)


def test_prelu_matches_exact_arithmetic_for_every_input_value():
    """every int8 input on every channel: x > 0 -> nearest(x * m / 2^rp), else nearest(slope * x / 2^rn),
    ties toward +inf, saturated"""
    c = 7
    slope = np.array([-128, -3, -1, 0, 1, 55, 127], np.float32)
    x = np.tile(np.arange(-128, 128, dtype=np.int8).reshape(1, 1, 256, 1), (2, c, 1, 1))
    for mp, rp, rn in [(1, 0, 0), (3, 1, 2), (200, 7, 5), (77, 4, 6)]:
        got = O.prelu_i8(x, slope, rp, mp, rn)
        for ch in range(c):
            for v in range(-128, 128):
                want = (sat8(nearest_ties_up(Fraction(v * mp, 1 << rp))) if v > 0 else
                        sat8(nearest_ties_up(Fraction(int(slope[ch]) * v, 1 << rn))))
                assert got[1, ch, v + 128, 0] == want, (mp, rp, rn, ch, v)


def test_scale_lut_reads_each_channels_table_at_the_unsigned_value():
    """every uint8 value on every channel equals plain numpy indexing table[c, x]; the tables are
    built the way the quantizer builds them (saturated nearest of idx * scale + bias)"""
    c = 5
    scale = np.array([0.5, 1.0, 0.017, 2.0, 0.25])
    bias = np.array([-64.0, -128.0, 3.0, -300.0, 0.4])
    idx = np.arange(256)
    table = np.clip(np.floor(idx[None, :] * scale[:, None] + bias[:, None] + 0.5), -128, 127).astype(np.float32)
    x = np.tile(idx.astype(np.uint8).reshape(1, 1, 16, 16), (2, c, 1, 1))
    x[1] = x[1, :, ::-1, ::-1]
    got = O.scale_lut_u8(x, table.reshape(-1))
    want = table.astype(np.int8)[np.arange(c)[None, :, None, None], x.astype(np.int64)]
    assert got.dtype == np.int8 and np.array_equal(got, want)
    # channel 1 is the identity shifted by 128: the unsigned byte reinterpreted as int8
    assert np.array_equal(got[:, 1], (x[:, 1].astype(np.int16) - 128).astype(np.int8))
