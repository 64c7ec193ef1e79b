"""The host-side quantisation arithmetic against independent mathematics: exact rationals for
the multiplier decompositions, reconstruction properties for the weight quantizers, 40-digit
decimal evaluation for the activation tables.  No GPU."""
import math
from decimal import Decimal, getcontext
from fractions import Fraction

import numpy as np
import pytest

from tpu_compiler_amd import capi, quantize as Q

getcontext().prec = 40


def expected_quantize_multiplier(m):
    """the TensorFlow Lite decomposition restated with exact rationals on math.frexp"""
    if m == 0:
        return 0, 0
    q, s = math.frexp(m)
    qf = math.floor(Fraction(q) * 2 ** 31 + Fraction(1, 2))     # round half away from zero, q > 0
    if qf == 2 ** 31:
        qf, s = 2 ** 30, s + 1
    if s < -31:
        return 0, 0
    return qf, s


def test_quantize_multiplier_known_answers_and_exact_sweep():
    assert Q.quantize_multiplier(0.5) == (1 << 30, 0)
    assert Q.quantize_multiplier(1.0) == (1 << 30, 1)
    assert Q.quantize_multiplier(0.75) == (3 << 29, 0)
    assert Q.quantize_multiplier(0.0) == (0, 0)
    assert Q.quantize_multiplier(1.0 - 2.0 ** -33) == (1 << 30, 1)      # rounds up to 2^31: renormalised
    assert Q.quantize_multiplier(2.0 ** -40) == (0, 0)                  # flushed: shift below -31
    assert Q.quantize_multiplier(2.0 ** -31) == (1 << 30, -30)
    rng = np.random.default_rng(0)
    values = [2.0 ** k for k in range(-31, 8)] + [np.nextafter(2.0 ** k, 0) for k in range(-20, 4)]
    values += list(np.exp(rng.uniform(math.log(1e-9), math.log(50.0), 3000)))
    values += [0.999999, 0.1, 1 / 3, 127 / 128]
    for m in values:
        m = float(m)
        q, s = Q.quantize_multiplier(m)
        assert (q, s) == expected_quantize_multiplier(m), m
        if q:
            assert (1 << 30) <= q < (1 << 31)
            assert abs(Fraction(m) - Fraction(q) * Fraction(2) ** (s - 31)) <= Fraction(2) ** (s - 32)
    with pytest.raises(capi.TpuHipError, match="negative"):
        Q.quantize_multiplier(-0.5)


def test_find_rshift_and_multiplier_both_forms():
    rng = np.random.default_rng(1)
    # 8-bit form: smallest rshift with qscale * 2^(rshift+1) >= max, multiplier = floor(qscale * 2^rshift)
    for qs in list(np.exp(rng.uniform(math.log(1e-6), math.log(126.0), 2000))) + [1.0, 0.5, 63.5, 127.0, 1e-3]:
        for mx in (127, 255):
            qs = float(qs)
            r, m = Q.find_rshift_and_multiplier(qs, False, mx)
            f = Fraction(qs)
            want_r = next(k for k in range(63) if f * 2 ** (k + 1) >= mx)
            assert (r, m) == (want_r, math.floor(f * 2 ** want_r)), (qs, mx)
            assert m >= (mx - 1) // 2 and (m < mx if r > 0 else m <= mx)
            assert Fraction(m, 2 ** r) <= f < Fraction(m + 1, 2 ** r)
    assert Q.find_rshift_and_multiplier(300.0, False, 127) == (0, 127)      # larger than the maximum
    assert Q.find_rshift_and_multiplier(1e-30, False, 127) == (0, 0)        # too small for any shift
    # 32-bit form: rshift = -shift of the decomposition, qscale >= 1 replaced by 0.999999
    for qs in [0.3, 0.9, 1e-4, 0.999999, 2.0 ** -7]:
        q, s = expected_quantize_multiplier(qs)
        assert Q.find_rshift_and_multiplier(qs, True) == (-s, q)
    assert Q.find_rshift_and_multiplier(1.0, True) == Q.find_rshift_and_multiplier(0.999999, True)
    assert Q.find_rshift_and_multiplier(17.0, True) == Q.find_rshift_and_multiplier(0.999999, True)


def _qscale_eff(rshift, mult):
    return Fraction(int(mult), 2 ** (31 + int(rshift)))


def test_conv_weight_quantizer_reconstructs_the_weights():
    rng = np.random.default_rng(2)
    oc, isz = 7, 45
    w = rng.normal(0, 0.2, (oc, 5, 3, 3)).astype(np.float32)
    w[3] *= 1e-3                                     # a nearly dead channel still gets full range
    b = rng.normal(0, 0.5, oc).astype(np.float32)
    thx, thy = 2.7, 5.1
    wq, bq, rs, mu = Q.quantize_conv(w, b, thx, thy)
    assert wq.dtype == np.float32 and np.array_equal(wq, np.rint(wq)) and np.array_equal(bq, np.rint(bq))
    for c in range(oc):
        maxw = np.float32(np.abs(w[c]).max())
        qs32 = np.float32(maxw * np.float32(thx)) / np.float32(np.float32(127.0) * np.float32(thy))   # float path
        r, m = Q.find_rshift_and_multiplier(float(qs32), True)
        assert (rs[c], mu[c]) == (r, m), c
        assert (1 << 30) <= m < (1 << 31)
        eff = _qscale_eff(r, m)
        assert abs(eff / Fraction(float(qs32)) - 1) < Fraction(1, 2 ** 30)
        # the largest weight lands on +-127 and every weight within half a step of its exact image
        assert np.abs(wq[c]).max() == 127
        scale = float(Fraction(float(np.float32(thx) / np.float32(thy))) / eff)
        assert np.abs(wq[c].reshape(-1) - w[c].reshape(-1).astype(np.float64) * scale).max() <= 0.5 + 1e-4
        exact_b = float(b[c]) * float(Fraction(float(np.float32(128.0) / np.float32(thy))) / eff)
        assert abs(bq[c] - exact_b) <= 0.5 + abs(exact_b) * 1e-6
    # without a bias nothing about the filter changes
    wq2, bq2, rs2, mu2 = Q.quantize_conv(w, None, thx, thy)
    assert bq2 is None and np.array_equal(wq2, wq) and np.array_equal(rs2, rs) and np.array_equal(mu2, mu)


def test_conv_weight_quantizer_special_cases():
    rng = np.random.default_rng(3)
    w = rng.normal(0, 0.2, (4, 18)).astype(np.float32)
    thx, thy = 1.0, 4.0
    # a bias too large for int32 at the filter's scale raises the channel's qscale: weights lose range
    b = np.array([0.0, 3.0e5, 0.0, 0.0], np.float32)
    wq, bq, rs, mu = Q.quantize_conv(w, b, thx, thy)
    wq0, _, rs0, mu0 = Q.quantize_conv(w, np.zeros(4, np.float32), thx, thy)
    assert np.abs(wq[1]).max() < 127 and _qscale_eff(rs[1], mu[1]) > _qscale_eff(rs0[1], mu0[1])
    assert abs(bq[1]) < 2 ** 31 and abs(bq[1]) > 0.97 * 2 ** 31
    for c in (0, 2, 3):
        assert np.array_equal(wq[c], wq0[c]) and rs[c] == rs0[c] and mu[c] == mu0[c]
    # given filter thresholds replace the measured maxima: values beyond them saturate
    ft = np.abs(w).max(axis=1).astype(np.float32) * np.float32(0.5)
    wq3, _, _, _ = Q.quantize_conv(w, None, thx, thy, filter_threshold=ft)
    for c in range(4):
        big = np.abs(w[c]) > ft[c] * 1.01
        assert big.any() and (np.abs(wq3[c][big]) >= 127).all() and wq3[c].min() >= -128 and wq3[c].max() <= 127
    # qscale >= 1 (output threshold tiny): clamped to 0.999999, the filter saturates instead of shifting left
    wq4, _, rs4, mu4 = Q.quantize_conv(w, None, 50.0, 0.01)
    r, m = Q.find_rshift_and_multiplier(0.999999, True)
    assert (rs4 == r).all() and (mu4 == m).all() and (np.abs(wq4) >= 127).mean() > 0.9
    with pytest.raises(capi.TpuHipError, match="bad argument"):
        capi.check(capi.bind(), capi.bind().tpuhip_quantize_conv_weights(None, None, 1, 1, 1.0, 1.0, None, None,
                                                                         None, None, None))


def test_fc_weight_quantizer_is_per_batch():
    rng = np.random.default_rng(4)
    w = rng.normal(0, 0.05, (10, 64)).astype(np.float32)
    b = rng.normal(0, 0.3, 10).astype(np.float32)
    thx, thy = 3.3, 9.0
    wq, bq, rs, mu = Q.quantize_fc(w, b, thx, thy)
    assert rs.shape == (1,) and mu.shape == (1,)
    maxw = np.float32(np.abs(w).max())
    qs32 = np.float32(maxw * np.float32(thx)) / np.float32(np.float32(127.0) * np.float32(thy))
    assert (rs[0], mu[0]) == Q.find_rshift_and_multiplier(float(qs32), True)
    eff = _qscale_eff(rs[0], mu[0])
    scale = float(Fraction(float(np.float32(thx) / np.float32(thy))) / eff)
    assert np.abs(wq).max() == 127 and np.abs(wq - w.astype(np.float64) * scale).max() <= 0.5 + 1e-4
    bscale = float(Fraction(float(np.float32(128.0) / np.float32(thy))) / eff)
    assert np.abs(bq - b.astype(np.float64) * bscale).max() <= 0.5 + np.abs(b * bscale).max() * 1e-6
    # two batches are quantized independently
    w2 = np.stack([w, w * 4]).astype(np.float32)
    wq2, _, rs2, mu2 = Q.quantize_fc(w2, None, thx, thy)
    assert np.array_equal(wq2[0], wq) and np.abs(wq2[1]).max() == 127
    assert _qscale_eff(rs2[1], mu2[1]) > 3.9 * _qscale_eff(rs2[0], mu2[0])


def test_rescale_of_weightless_ops():
    # eltwise add of two inputs onto one output threshold: one shift, a multiplier per input
    rs, mu = Q.quantize_rescale([2.0, 3.5], 4.0)
    r = int(rs[0])
    qs = [np.float32(2.0) / np.float32(4.0), np.float32(3.5) / np.float32(4.0)]
    assert r == next(k for k in range(63) if Fraction(float(max(qs))) * 2 ** (k + 1) >= 127)
    for q, m in zip(qs, mu):
        assert m == math.floor(Fraction(float(q)) * 2 ** r)
    assert 63 <= mu.max() < 127
    # global average pool 7x7: the 1/49 is part of the scale
    rs, mu = Q.quantize_rescale([3.0], 3.0, divisor=49)
    q = np.float32(np.float32(3.0) / np.float32(3.0)) / np.float32(49)
    assert mu[0] == math.floor(Fraction(float(q)) * 2 ** int(rs[0])) and 63 <= mu[0] < 127
    assert abs(mu[0] / 2 ** rs[0] * 49 - 1) < 0.02
    # coefficients scale the inputs; a negative one has no int8 form here
    rs, mu = Q.quantize_rescale([2.0, 2.0], 4.0, coeff=[1.0, 0.5])
    assert mu[0] == 2 * mu[1] or mu[0] == 2 * mu[1] + 1
    with pytest.raises(capi.TpuHipError, match="negative scale"):
        Q.quantize_rescale([2.0, 2.0], 4.0, coeff=[1.0, -1.0])


def test_leaky_relu_parameters():
    p = Q.quantize_leaky_relu(0.1, 3.0, 3.0)
    assert (p["rshift_pos"][0], p["multiplier_pos"][0]) == (0, 1)           # equal thresholds: no scale
    assert (p["rshift_neg"][0], p["multiplier_neg"][0]) == Q.find_rshift_and_multiplier(
        float(np.float32(abs(float(np.float32(3.0) / np.float32(3.0)) * np.float32(0.1)))), False)
    p = Q.quantize_leaky_relu(0.1, 2.0, 3.0)
    qpos = float(np.float32(2.0) / np.float32(3.0))
    assert (p["rshift_pos"][0], p["multiplier_pos"][0]) == Q.find_rshift_and_multiplier(qpos, False)
    assert abs(p["multiplier_neg"][0] / 2 ** p["rshift_neg"][0] - qpos * 0.1) < qpos * 0.1 / 60


def _index(i, thx):
    """the table argument the way it is formed: (int8 * float32 threshold) in float32, / 127 in double"""
    v = i if i < 128 else i - 256
    return v, Decimal(float(np.float32(v) * np.float32(thx))) / Decimal(127)


@pytest.mark.parametrize("kind", ["sigmoid", "tanh", "exp", "elu", "swish", "softplus", "log", "mish"])
def test_activation_tables_against_40_digit_arithmetic(kind):
    thx, thy, scale, bias = 5.3, (1.0 if kind in ("sigmoid", "tanh") else 6.1), 1.0, 0.0
    if kind == "exp":
        thx, thy = 2.0, 7.5
    table = Q.quantize_lut_table(kind, thx, thy, scale, bias)
    margin = Decimal("1e-2") if kind in ("softplus", "mish") else Decimal("1e-9")    # these run in float32
    decided = 0
    for i in range(256):
        v, x = _index(i, thx)
        if kind == "log" and v <= 0:
            assert (np.isnan(table[i]) if v < 0 else table[i] == -128), i
            continue
        if kind == "sigmoid":
            y = Decimal(1) / (1 + (-x).exp())
        elif kind == "tanh":
            e = (2 * x).exp()
            y = (e - 1) / (e + 1)
        elif kind == "exp":
            y = x.exp()
        elif kind == "elu":
            y = x if x >= 0 else x.exp() - 1
        elif kind == "swish":
            y = x / (1 + (-x).exp())
        elif kind == "softplus":
            y = (x.exp() + 1).ln()
        elif kind == "mish":
            e = (2 * (x.exp() + 1).ln()).exp()          # x * tanh(softplus(x))
            y = x * (e - 1) / (e + 1)
        else:
            y = x.ln()
        t = y * Decimal(127) / Decimal(float(np.float32(thy)))
        want = max(-128, min(127, math.floor(t + Decimal("0.5"))))
        frac = (t + Decimal("0.5")) - math.floor(t + Decimal("0.5"))
        if min(frac, 1 - frac) < margin:
            continue                            # too close to a rounding tie to call
        decided += 1
        assert table[i] == want, (kind, i, v, float(t))
    assert decided >= (120 if kind == "log" else 240 if kind == "mish" else 250)
    assert len(np.unique(table[~np.isnan(table)])) > 20


def test_power_tables_and_errors():
    thx, thy = 4.0, 9.0
    t = Q.quantize_lut_table("pow", thx, thy, coeff=2.0)
    for i in range(256):
        v = i if i < 128 else i - 256
        exact = Fraction(127) / Fraction(float(np.float32(thy))) * (Fraction(float(np.float32(thx))) / 127) ** 2 * v * v
        want = max(-128, min(127, math.floor(exact + Fraction(1, 2))))
        if abs((exact + Fraction(1, 2)) % 1) > 1e-9 and abs((exact + Fraction(1, 2)) % 1 - 1) > 1e-9:
            assert t[i] == want, i
    t = Q.quantize_lut_table("pow", thx, thy, coeff=0.5)
    assert (t[128:] == 0).all() and t[0] == 0 and t[127] > t[64] > t[1] > 0      # no root of a negative input
    t = Q.quantize_lut_table("pow", thx, thy, coeff=-1.0)
    assert t[0] == 127 and t[1] == 127 and t[255] == -128 and t[127] > 0
    with pytest.raises(capi.TpuHipError, match="unknown kind"):
        capi.check(capi.bind(), capi.bind().tpuhip_quantize_lut_table(99, 1.0, 1.0, 1.0, 0.0, 0.0,
                                                                      np.empty(256, np.float32).ctypes.data))
