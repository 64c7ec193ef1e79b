"""Pins the oracle's tensor ops against library routines (torch float64 conv /
max-pool, numpy repeat / concatenate), brute-force loops on tiny shapes, exact
rational arithmetic and exhaustive 256-entry sweeps."""
import itertools
import math
from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle_lib as O


def rnd_i8(rng, shape, lo=-128, hi=127):
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int64).astype(np.int8)


def brute_conv(x, w, g, stride, pads, dil, ins, out_hw):
    n, ic, ih, iw = x.shape
    oc, icg, kh, kw = w.shape
    oh, ow = out_hw
    ocg = oc // g
    # dilate the input exactly as my_dilateActivation does: zeros between samples
    ihd, iwd = (ih - 1) * (ins[0] + 1) + 1, (iw - 1) * (ins[1] + 1) + 1
    xd = np.zeros((n, ic, ihd, iwd), np.int64)
    xd[:, :, ::ins[0] + 1, ::ins[1] + 1] = x
    acc = np.zeros((n, oc, oh, ow), np.int64)
    for b, o, y, xx in itertools.product(range(n), range(oc), range(oh), range(ow)):
        s = 0
        for c, i, j in itertools.product(range(icg), range(kh), range(kw)):
            hh = y * stride[0] - pads[0] + i * dil[0]
            ww = xx * stride[1] - pads[2] + j * dil[1]
            if 0 <= hh < ihd and 0 <= ww < iwd:
                s += int(xd[b, (o // ocg) * icg + c, hh, ww]) * int(w[o, c, i, j])
        acc[b, o, y, xx] = s
    return acc


CONV_TINY = [
    # n ic ih iw oc g kh kw stride pads(t,b,l,r) dil ins
    (1, 3, 5, 6, 4, 1, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), (0, 0)),
    (2, 4, 7, 5, 6, 2, 3, 2, (2, 1), (0, 1, 2, 0), (1, 1), (0, 0)),
    (1, 4, 6, 6, 4, 4, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), (0, 0)),   # depthwise
    (1, 2, 9, 8, 3, 1, 3, 3, (1, 2), (2, 2, 2, 2), (2, 2), (0, 0)),   # dilation
    (1, 2, 4, 4, 3, 1, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), (1, 1)),   # inserted zeros
    (2, 6, 5, 5, 6, 3, 1, 1, (2, 2), (0, 0, 0, 0), (1, 1), (0, 0)),   # grouped 1x1 s2
    (1, 3, 8, 8, 2, 1, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1), (0, 0)),   # 7x7 s2 p3
    (1, 2, 5, 7, 2, 1, 2, 3, (1, 1), (0, 1, 1, 1), (1, 1), (0, 2)),
]


@pytest.mark.parametrize("cfg", CONV_TINY)
def test_conv_acc_brute_force(cfg):
    n, ic, ih, iw, oc, g, kh, kw, stride, pads, dil, ins = cfg
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_i8(rng, (oc, ic // g, kh, kw))
    d = O.make_conv_desc(x.shape, w.shape, g, stride, pads, dil, ins)
    want = brute_conv(x, w, g, stride, pads, dil, ins, (d.oh, d.ow))
    got = O.conv2d_acc(x, w, d)
    assert np.array_equal(got.astype(np.int64), want)


CONV_TORCH = [
    (2, 64, 28, 28, 64, 1, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1)),
    (1, 64, 56, 56, 64, 1, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1)),       # cfg1 shape
    (2, 3, 64, 64, 16, 1, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1)),
    (2, 32, 20, 20, 32, 32, 3, 3, (2, 2), (1, 1, 1, 1), (1, 1)),      # depthwise s2
    (1, 48, 14, 14, 96, 1, 1, 1, (2, 2), (0, 0, 0, 0), (1, 1)),
    (1, 16, 19, 19, 24, 2, 3, 3, (1, 1), (2, 2, 2, 2), (2, 2)),
]


@pytest.mark.parametrize("cfg", CONV_TORCH)
def test_conv_acc_vs_torch_float64(cfg):
    n, ic, ih, iw, oc, g, kh, kw, stride, pads, dil = cfg
    assert pads[0] == pads[1] and pads[2] == pads[3]
    rng = np.random.default_rng(ic * 131 + oc)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_i8(rng, (oc, ic // g, kh, kw))
    d = O.make_conv_desc(x.shape, w.shape, g, stride, pads, dil)
    got = O.conv2d_acc(x, w, d)
    ref = F.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(w.astype(np.float64)),
                   None, stride, (pads[0], pads[2]), dil, g).numpy()
    assert np.array_equal(got.astype(np.float64), ref)


def test_conv_asymmetric_padding_vs_torch_pad():
    rng = np.random.default_rng(8)
    x = rnd_i8(rng, (1, 8, 13, 11))
    w = rnd_i8(rng, (8, 8, 3, 3))
    pads = (0, 1, 2, 1)  # t, b, l, r
    d = O.make_conv_desc(x.shape, w.shape, 1, (2, 2), pads)
    xp = F.pad(torch.from_numpy(x.astype(np.float64)), (pads[2], pads[3], pads[0], pads[1]))
    ref = F.conv2d(xp, torch.from_numpy(w.astype(np.float64)), None, (2, 2)).numpy()
    assert np.array_equal(O.conv2d_acc(x, w, d).astype(np.float64), ref)


def test_fp32_dataflow_equals_int32_under_guard():
    # the reference accumulates in fp32; below 2^24 that is exact in any order
    rng = np.random.default_rng(21)
    x = rnd_i8(rng, (1, 64, 14, 14))
    w = np.clip(np.rint(rng.normal(0, 32, (32, 64, 3, 3))), -127, 127).astype(np.int8)
    d = O.make_conv_desc(x.shape, w.shape, 1, (1, 1), (1, 1, 1, 1))
    guard = O.conv2d_guard(x, w, d)
    assert guard < (1 << 24)
    a_i = O.conv2d_acc(x, w, d)
    a_f = O.conv2d_acc_f32(x.astype(np.float32), w.astype(np.float32), d)
    assert np.array_equal(a_f, a_i.astype(np.float32))
    # the guard value itself: compare with an int64 conv of absolute values
    ref = F.conv2d(torch.from_numpy(np.abs(x.astype(np.float64))),
                   torch.from_numpy(np.abs(w.astype(np.float64))), None, 1, 1).numpy()
    assert guard == int(ref.max())


def test_fp32_dataflow_can_differ_beyond_guard():
    # all-extreme operands with K = 4608 exceed 2^24: the guard must say so
    x = np.full((1, 512, 3, 3), -128, np.int8)
    w = np.full((1, 512, 3, 3), -127, np.int8)
    d = O.make_conv_desc(x.shape, w.shape, 1, (1, 1), (1, 1, 1, 1))
    assert O.conv2d_guard(x, w, d) == 512 * 9 * 128 * 127 > (1 << 24)


def qdm_exact(v, m, r):
    s1 = math.floor(Fraction(v * m, 1 << 31) + Fraction(1, 2))
    a = abs(Fraction(s1, 1 << r))
    s2 = (1 if s1 >= 0 else -1) * math.floor(a + Fraction(1, 2)) if r else s1
    return max(-128, min(127, s2))


def test_requant_per_channel_layout_bias_relu():
    rng = np.random.default_rng(4)
    n, oc, oh, ow = 2, 5, 3, 4
    acc = rng.integers(-(1 << 20), 1 << 20, (n, oc, oh, ow)).astype(np.int32)
    bias = rng.integers(-4096, 4097, oc).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
    rsh = rng.integers(6, 14, oc).astype(np.float32)
    for relu in (False, True):
        got = O.requant_per_channel(acc, bias, rsh, mult, relu)
        for b, c, i, j in itertools.product(range(n), range(oc), range(oh), range(ow)):
            want = qdm_exact(int(acc[b, c, i, j]) + int(bias[c]), int(mult[c]), int(rsh[c]))
            if relu:
                want = max(want, 0)
            assert got[b, c, i, j] == want
    # no bias pointer == zero bias
    got0 = O.requant_per_channel(acc, None, rsh, mult, False)
    gotz = O.requant_per_channel(acc, np.zeros(oc), rsh, mult, False)
    assert np.array_equal(got0, gotz)


def test_requant_uses_float32_rounded_multiplier():
    acc = np.array([[[[1 << 20]]]], np.int32)
    m_int = (1 << 30) + 65  # not a float32: rounds to 2^30 + 128
    got = O.requant_per_channel(acc, None, [8], [np.float32(m_int)], False)
    assert got[0, 0, 0, 0] == qdm_exact(1 << 20, int(np.float32(m_int)), 8)


def test_conv2d_i8_is_acc_then_requant_and_without_bias_ignores_bias():
    rng = np.random.default_rng(17)
    x = rnd_i8(rng, (2, 8, 6, 6))
    w = rnd_i8(rng, (4, 8, 3, 3), -40, 40)
    bias = rng.integers(-4096, 4097, 4).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, 4) * 128).astype(np.float32)
    rsh = rng.integers(6, 10, 4).astype(np.float32)
    d = O.make_conv_desc(x.shape, w.shape, 1, (1, 1), (1, 1, 1, 1), do_relu=True)
    y = O.conv2d_i8(x, w, bias, rsh, mult, d)
    ref = F.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(w.astype(np.float64)),
                   None, 1, 1).numpy().astype(np.int64)
    for idx in np.ndindex(*y.shape):
        want = max(0, qdm_exact(int(ref[idx]) + int(bias[idx[1]]), int(mult[idx[1]]), int(rsh[idx[1]])))
        assert y[idx] == want
    d2 = O.make_conv_desc(x.shape, w.shape, 1, (1, 1), (1, 1, 1, 1), do_relu=True, with_bias=False)
    y2 = O.conv2d_i8(x, w, bias, rsh, mult, d2)
    y3 = O.conv2d_i8(x, w, np.zeros(4), rsh, mult, d)
    assert np.array_equal(y2, y3)


def test_fc_per_batch_requant_bias_before_relu():
    rng = np.random.default_rng(23)
    batch, m, k, n = 2, 3, 40, 5
    x = rnd_i8(rng, (batch, m, k))
    w = rnd_i8(rng, (batch, n, k))
    bias = rng.integers(-3000, 3000, (batch, n)).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, batch) * 128).astype(np.float32)
    rsh = np.array([7, 9], np.float32)
    for relu in (False, True):
        y = O.fc_i8(x, w, bias, rsh, mult, batch, m, k, n, relu)
        for b, i, j in itertools.product(range(batch), range(m), range(n)):
            s = int(np.dot(x[b, i].astype(np.int64), w[b, j].astype(np.int64))) + int(bias[b, j])
            if relu:
                s = max(s, 0)
            assert y[b, i, j] == qdm_exact(s, int(mult[b]), int(rsh[b]))
    assert O.fc_guard(x, w, bias, batch, m, k, n) < (1 << 24)


@pytest.mark.parametrize("ltrans,otrans", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_fc_batched_and_transposed_vs_numpy_einsum(ltrans, otrans):
    """core/fullyconnected.cpp:52-88: the permutes are numpy transposes, the matmuls an int64 einsum;
    the requant pair of an element is picked by its position in the final layout (block f // (m*n)),
    which differs from its matmul's batch index once the output is permuted"""
    rng = np.random.default_rng(31 + 2 * ltrans + otrans)
    bh, bl, m, k, n = 2, 3, 4, 24, 5
    batch = bh * bl
    x_l = rnd_i8(rng, (bh, m, bl, k) if ltrans else (batch, m, k))       # logical input
    w = rnd_i8(rng, (batch, n, k))
    bias = rng.integers(-3000, 3000, (batch, n)).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, batch) * 128).astype(np.float32)
    rsh = rng.integers(5, 10, batch).astype(np.float32)
    xb = x_l.transpose(0, 2, 1, 3).reshape(batch, m, k) if ltrans else x_l
    sums = np.einsum("bmk,bnk->bmn", xb.astype(np.int64), w.astype(np.int64)) + bias.astype(np.int64)[:, None, :]
    if otrans:
        sums = sums.reshape(bh, bl, m, n).transpose(0, 2, 1, 3)
    flat = sums.reshape(-1)
    for relu in (0, 1):
        y = O.fc_batched_i8(x_l, w, bias, rsh, mult, bh, bl, m, k, n, ltrans, otrans, relu)
        for f, s in enumerate(flat):
            s = max(int(s), 0) if relu else int(s)
            i = f // (m * n)
            assert y[f] == qdm_exact(s, int(mult[i]), int(rsh[i])), (f, relu)
    if not ltrans and not otrans:
        assert np.array_equal(O.fc_batched_i8(x_l, w, bias, rsh, mult, bh, bl, m, k, n, 0, 0, 1),
                              O.fc_i8(x_l, w, bias, rsh, mult, batch, m, k, n, True).reshape(-1))


def test_eltwise_add_closed_form():
    rng = np.random.default_rng(29)
    xs = [rnd_i8(rng, (2, 3, 4, 5)) for _ in range(3)]
    mult = np.array([5, -3, 7], np.float32)
    for rs, relu in itertools.product((0, 1, 3, 6), (False, True)):
        y = O.eltwise_add_i8(xs, mult, [rs], relu)
        s = sum(a.astype(np.int64) * int(m) for a, m in zip(xs, mult))
        if relu:
            s = np.maximum(s, 0)
        want = np.clip((s + ((1 << rs) >> 1)) >> rs, -128, 127)  # floor(s/2^r + 1/2)
        assert np.array_equal(y.astype(np.int64), want)


def test_eltwise_multiplier_is_truncated_to_int8():
    x = np.array([10, -10], np.int8)
    y = O.eltwise_add_i8([x], [3.9], [0], False)   # (int8_t)3.9 == 3
    assert list(y) == [30, -30]


@pytest.mark.parametrize("k,s,pads,shape", [
    ((3, 3), (2, 2), (0, 1, 0, 1), (2, 4, 12, 12)),   # the Caffe ceil-mode maxpool of ResNet-50
    ((3, 3), (2, 2), (1, 1, 1, 1), (1, 3, 9, 11)),
    ((2, 2), (2, 2), (0, 0, 0, 0), (1, 5, 8, 8)),
    ((3, 2), (1, 2), (1, 0, 0, 1), (1, 2, 7, 9)),
])
def test_pool_max_vs_torch(k, s, pads, shape):
    rng = np.random.default_rng(sum(shape))
    x = rnd_i8(rng, shape)
    d = O.make_pool_desc(shape, k, s, pads)
    xp = F.pad(torch.from_numpy(x.astype(np.float64)), (pads[2], pads[3], pads[0], pads[1]),
               value=float("-inf"))
    ref = F.max_pool2d(xp, k, s).numpy()
    assert np.array_equal(O.pool_max_i8(x, d).astype(np.float64), ref)


@pytest.mark.parametrize("k,s,pads,shape", [
    ((7, 7), (1, 1), (0, 0, 0, 0), (2, 16, 7, 7)),    # global average
    ((3, 3), (2, 2), (1, 1, 1, 1), (1, 4, 9, 9)),     # padding counts as zeros
    ((2, 2), (2, 2), (0, 0, 0, 0), (1, 3, 6, 6)),
])
def test_pool_avg_window_sum_then_half_up(k, s, pads, shape):
    rng = np.random.default_rng(sum(shape) + 1)
    x = rnd_i8(rng, shape)
    d = O.make_pool_desc(shape, k, s, pads)
    xp = F.pad(torch.from_numpy(x.astype(np.float64)), (pads[2], pads[3], pads[0], pads[1]))
    sums = (F.avg_pool2d(xp, k, s) * (k[0] * k[1])).round().numpy().astype(np.int64)
    for mult, rs in ((167, 13), (1, 0), (255, 14), (81, 12)):
        y = O.pool_avg_i8(x, d, rs, mult)
        want = np.clip(np.floor_divide(sums * mult + ((1 << rs) >> 1), 1 << rs), -128, 127)
        assert np.array_equal(y.astype(np.int64), want)


def half_up(fr):
    return max(-128, min(127, math.floor(fr + Fraction(1, 2))))


def test_leaky_relu_exhaustive():
    x = np.arange(-128, 128, dtype=np.int16).astype(np.int8)
    for rp, mp, rn, mn in ((0, 1, 7, 13), (5, 33, 10, 102), (0, 0, 6, 6), (3, 9, 0, 1)):
        y = O.leaky_relu_i8(x, rp, mp, rn, mn)
        for xi, yi in zip(x.tolist(), y.tolist()):
            if xi > 0:
                want = half_up(Fraction(xi * mp, 1 << rp)) if mp != 0 else xi
            else:
                want = half_up(Fraction(xi * mn, 1 << rn))
            assert yi == want, (xi, rp, mp, rn, mn)


def test_lut_index_is_twos_complement_byte():
    table = np.arange(256, dtype=np.float32) - 128          # table[i] = i - 128
    x = np.arange(-128, 128, dtype=np.int16).astype(np.int8)
    y = O.lut_i8(x, table)
    want = (x.view(np.uint8).astype(np.int16) - 128).astype(np.int8)
    assert np.array_equal(y, want)
    # x=0 -> entry 0 ; x=-128 -> entry 128 ; x=-1 -> entry 255 ; x=127 -> entry 127
    assert y[128] == -128 and y[0] == 0 and y[127] == 127 and y[255] == -1


def test_relu_and_clip():
    x = np.arange(-128, 128, dtype=np.int16).astype(np.int8)
    assert np.array_equal(O.relu_i8(x), np.maximum(x, 0))
    y = O.clip_i8(x, 0, 93, 0, 1)
    assert np.array_equal(y, np.clip(x, 0, 93))
    y = O.clip_i8(x, -20, 50, 2, 3)
    want = [half_up(Fraction(min(max(int(v), -20), 50) * 3, 4)) for v in x]
    assert y.tolist() == want


def test_upsample_vs_numpy_repeat():
    rng = np.random.default_rng(31)
    x = rnd_i8(rng, (2, 3, 5, 4))
    for sh, sw in ((2, 2), (1, 3), (3, 1)):
        want = np.repeat(np.repeat(x, sh, axis=2), sw, axis=3)
        assert np.array_equal(O.upsample_i8(x, sh, sw), want)


def test_concat_vs_numpy_and_requant():
    rng = np.random.default_rng(37)
    a, b, c = rnd_i8(rng, (2, 3, 4, 4)), rnd_i8(rng, (2, 5, 4, 4)), rnd_i8(rng, (2, 1, 4, 4))
    assert np.array_equal(O.concat_i8([a, b, c], 1), np.concatenate([a, b, c], 1))
    a2, b2 = rnd_i8(rng, (2, 3, 4, 2)), rnd_i8(rng, (2, 3, 4, 5))
    assert np.array_equal(O.concat_i8([a2, b2], 3), np.concatenate([a2, b2], 3))
    y = O.concat_i8([a, b], 1, rshift=[0, 3], multiplier=[1, 5], do_relu=True)
    bq = np.clip((b.astype(np.int64) * 5 + 4) >> 3, -128, 127)
    want = np.maximum(np.concatenate([a.astype(np.int64), bq], 1), 0)
    assert np.array_equal(y.astype(np.int64), want)


def lrn_by_definition(x, local_size, sq, pw, sum_rshift, lrn_rshift, q0, q1):
    """the INT8 LRN as exact integer arithmetic written from the definition: window sum of the
    squares table over the channels, one rounding shift to the index, one to the result"""
    n, c, h, w = x.shape
    sqv = np.asarray(sq, np.int64)[x.astype(np.uint8)]
    pre = (local_size - 1) // 2
    pad = np.zeros((n, c + local_size - 1, h, w), np.int64)
    pad[:, pre:pre + c] = sqv
    s = sum(pad[:, k:k + c] for k in range(local_size)) * q0
    t = np.clip((s + ((1 << sum_rshift) >> 1)) >> sum_rshift, 0, 255)
    m = np.asarray(pw, np.int64)[t] * x.astype(np.int64) * q1
    return np.clip((m + ((1 << lrn_rshift) >> 1)) >> lrn_rshift, -128, 127).astype(np.int8)


@pytest.mark.parametrize("local_size,sum_rshift,lrn_rshift,q0,q1", [(5, 8, 9, 120, 93), (3, 0, 0, 1, 1),
                                                                     (1, 4, 12, 255, 255), (4, 10, 7, 77, 40)])
def test_lrn_float_restatement_equals_the_integer_definition(local_size, sum_rshift, lrn_rshift, q0, q1):
    """the oracle keeps the reference's float running sums; under the exactness bounds the result
    must equal plain integer arithmetic, negative inputs (which index the upper table half) included"""
    rng = np.random.default_rng(local_size * 7 + q0)
    x = rng.integers(-128, 128, (2, 11, 4, 3)).astype(np.int8)
    x[0, :, 0, 0] = 127
    x[1, :, 0, 0] = -128
    sq = rng.integers(0, 256, 256)
    pw = rng.integers(0, 256, 256)
    if lrn_rshift == 0:
        pw = pw % 3
    got = O.lrn_i8(x, local_size, sq, pw, sum_rshift, lrn_rshift, q0, q1)
    want = lrn_by_definition(x, local_size, sq, pw, sum_rshift, lrn_rshift, q0, q1)
    assert np.array_equal(got, want)
    assert len(np.unique(got)) > 3


def test_lrn_with_realistic_tables_tracks_the_float_formula():
    """tables as the quantiser builds them (QuantizeInt8.cpp:299-329) for a ReLU-ed input: the INT8
    result must follow x / (k + alpha/n * sum x^2)^beta"""
    rng = np.random.default_rng(2)
    thx, thy, alpha, beta, k, n_ = 4.0, 4.2, 1e-2, 0.75, 1.0, 5
    xf = np.abs(rng.normal(0, 1.2, (1, 16, 6, 6))).clip(0, thx)
    x = np.clip(np.floor(xf * 128 / thx + 0.5), -128, 127).astype(np.int8)
    sq_thy, sumsq_thy = alpha / n_ * thx * thx, alpha * thx * thx * 1.0
    scale_thy = k ** -beta
    idx = np.arange(256)
    sq = np.minimum(np.floor((thx / 128.0 * idx) ** 2 * 256.0 / sq_thy * alpha / n_ + 0.5), 255)
    pw = np.minimum(np.floor((idx / (256.0 / sumsq_thy) + k) ** -beta * (256.0 / scale_thy) + 0.5), 255)
    # sum of squares tables -> index: sq_thy / sumsq_thy as quant0 / 2^shift; result: thx*scale_thy/(thy*256)
    q0, r0 = int(round(sq_thy / sumsq_thy * 2 ** 12)), 12
    q1, r1 = int(round(thx * scale_thy / (thy * 256.0) * 2 ** 14)), 14
    got = O.lrn_i8(x, n_, sq, pw, r0, r1, q0, q1).astype(np.float64) * thy / 128
    xr = x.astype(np.float64) * thx / 128
    pad = np.zeros((1, 16 + n_ - 1, 6, 6))
    pad[:, 2:18] = xr ** 2
    ref = xr / (k + alpha / n_ * sum(pad[:, j:j + 16] for j in range(n_))) ** beta
    assert np.abs(got - ref).max() < 0.05 * thy


@pytest.mark.parametrize("kind", ["mean", "sum", "max", "min"])
@pytest.mark.parametrize("axes", [[2, 3], [1], [1, 2, 3], [3]])
def test_reduce_is_numpy_reduction_then_the_float_requant(kind, axes):
    rng = np.random.default_rng(len(axes) * 11 + len(kind))
    x = rng.integers(-128, 128, (2, 7, 5, 6)).astype(np.int8)
    fn = {"mean": np.sum, "sum": np.sum, "max": np.max, "min": np.min}[kind]     # an INT8 mean is a sum
    red = fn(x.astype(np.int64), axis=tuple(axes), keepdims=True)
    for rshift, mult in [(7, 55), (0, 3), (12, 200)] + ([(0, 1)] if kind in ("max", "min") else []):
        got = O.reduce_i8(kind, x, axes, red.shape, rshift, mult)
        if (rshift, mult) == (0, 1):
            want = red
        else:
            # float product, float quotient, floor(f + 0.5), clamp: all exact here (|sum * mult| < 2^24)
            want = np.clip(np.floor(red.astype(np.float64) * mult / (1 << rshift) + 0.5), -128, 127)
        assert np.array_equal(got, want), (rshift, mult)
    # without the reduced axes in the shape the bytes are the same
    squeezed = tuple(d for k, d in enumerate(red.shape) if k not in axes)
    assert np.array_equal(O.reduce_i8(kind, x, axes, squeezed, 7, 55).ravel(),
                          O.reduce_i8(kind, x, axes, red.shape, 7, 55).ravel())
