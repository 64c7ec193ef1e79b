"""Pins the oracle's data movement ops against numpy / torch routines that define the same
rearrangements independently (np.pad, slicing, transpose, tile, flip, reshape chains,
torch.pixel_shuffle)."""
import numpy as np
import pytest
import torch

import oracle_lib as O


def rnd(shape, seed=0):
    return np.random.default_rng(seed).integers(-128, 128, shape).astype(np.int8)


def test_pad_constant_is_zero_padding_and_negative_pads_cut():
    x = rnd((2, 3, 5, 4))
    got = O.move_i8("pad_const", x, [0, 1, 2, 3, 1, 0, 4, 1])
    assert np.array_equal(got, np.pad(x, [(0, 1), (1, 0), (2, 4), (3, 1)]))
    got = O.move_i8("pad_const", x, [0, -1, 2, -2, 0, 1, -1, 0])     # cut c at the front, w twice, h at the end
    want = np.pad(x[:, 1:, :4, 2:], [(0, 0), (0, 1), (2, 0), (0, 0)])
    assert np.array_equal(got, want)


def test_pad_edge_replicates_borders():
    x = rnd((2, 3, 5, 4), 1)
    got = O.move_i8("pad_edge", x, [0, 0, 2, 1, 0, 0, 3, 4])
    assert np.array_equal(got, np.pad(x, [(0, 0), (0, 0), (2, 3), (1, 4)], mode="edge"))


def test_crop_with_offsets_and_steps():
    x = rnd((3, 7, 9, 8), 2)
    got = O.move_i8("crop", x, [1, 2, 0, 3, 1, 1, 1, 1], out_shape=(2, 4, 9, 5))
    assert np.array_equal(got, x[1:3, 2:6, :, 3:8])
    got = O.move_i8("crop", x, [0, 1, 2, 0, 2, 3, 2, 4], out_shape=(2, 2, 4, 2))
    assert np.array_equal(got, x[0::2, 1::3, 2::2, 0::4][:2, :2, :4, :2])


@pytest.mark.parametrize("order", [(0, 2, 3, 1), (0, 3, 1, 2), (1, 0, 2, 3), (3, 2, 1, 0), (0, 1, 3, 2)])
def test_permute_is_numpy_transpose(order):
    x = rnd((2, 3, 5, 4), 3)
    assert np.array_equal(O.move_i8("permute", x, order), np.transpose(x, order))


def test_reorg_is_space_to_depth_with_the_block_offset_outermost():
    x = rnd((2, 3, 6, 4), 4)
    b, c, h, w = x.shape
    s = 2
    want = x.reshape(b, c, h // s, s, w // s, s).transpose(0, 3, 5, 1, 2, 4).reshape(b, s * s * c, h // s, w // s)
    assert np.array_equal(O.move_i8("reorg", x, [s]), want)


@pytest.mark.parametrize("axis", [0, 1, 2, 3])
def test_tile_and_reverse(axis):
    x = rnd((2, 3, 5, 4), 5)
    reps = [1, 1, 1, 1]
    reps[axis] = 3
    assert np.array_equal(O.move_i8("tile", x, [axis, 3]), np.tile(x, reps))
    assert np.array_equal(O.move_i8("reverse", x, [axis]), np.flip(x, axis))


def test_shuffle_channel_is_group_transpose():
    x = rnd((2, 12, 3, 4), 6)
    g = 3
    want = x.reshape(2, g, 12 // g, 3, 4).transpose(0, 2, 1, 3, 4).reshape(x.shape)
    assert np.array_equal(O.move_i8("shuffle_channel", x, [g]), want)


def test_swap_channel_is_fancy_indexing_of_the_channel_axis():
    rng = np.random.default_rng(3)
    x = rng.integers(-128, 128, (2, 3, 5, 4)).astype(np.int8)
    for order in ([2, 1, 0], [0, 1, 2], [1, 1, 2]):          # a repeat is legal: frames are copied
        assert np.array_equal(O.move_i8("swap_channel", x, order), x[:, order])


def test_dilate_is_a_strided_scatter_into_the_fill_value():
    x = rnd((2, 3, 4, 5), 8)
    for ins_w, ins_h, fill in [(1, 2, -7), (0, 3, 0), (2, 0, 127), (0, 0, 1)]:
        want = np.full((2, 3, (4 - 1) * (ins_h + 1) + 1, (5 - 1) * (ins_w + 1) + 1), fill, np.int8)
        want[:, :, ::ins_h + 1, ::ins_w + 1] = x
        assert np.array_equal(O.move_i8("dilate", x, [ins_w, ins_h, fill]), want), (ins_w, ins_h, fill)


def test_reflection_pad_is_numpy_reflect_on_the_last_axis():
    x = rnd((2, 3, 4, 6), 9)
    for left, right in [(0, 0), (2, 0), (0, 3), (5, 5), (1, 4)]:
        want = np.pad(x, ((0, 0), (0, 0), (0, 0), (left, right)), mode="reflect")
        assert np.array_equal(O.move_i8("reflection_pad", x, [left, right]), want), (left, right)


def test_zero_mask_and_mul_const_on_every_byte():
    x = np.arange(-128, 128).astype(np.int8).reshape(1, 256, 1, 1)
    xi = x.astype(np.int64)
    assert np.array_equal(O.zero_mask_i8(x, True), np.where(xi != 0, 127, 0))
    assert np.array_equal(O.zero_mask_i8(x, False), np.where(xi == 0, 127, 0))
    # the three constants the quantisation pass leaves, and fractions for the rounding rule:
    # nearest, ties to even on the magnitude (numpy's rint), saturated; -(-128) saturates to 127
    for c in (1.0, -1.0, 0.0, 0.5, -0.5, 1.5, 0.3):
        want = np.clip(np.rint(xi.astype(np.float32) * np.float32(c)), -128, 127)
        assert np.array_equal(O.mul_const_i8(x, c), want), c
        assert np.array_equal(O.mul_const_i8(x, c, True), np.maximum(want, 0)), c
    assert O.mul_const_i8(x, -1.0).ravel()[0] == 127
    assert O.mul_const_i8(x, 0.5).ravel()[128 + 1] == 0 and O.mul_const_i8(x, 0.5).ravel()[128 + 3] == 2


def test_depth_to_space_both_modes():
    x = rnd((2, 12, 3, 4), 7)
    r = 2
    crd = torch.pixel_shuffle(torch.from_numpy(x.astype(np.int32)), r).numpy().astype(np.int8)
    assert np.array_equal(O.move_i8("depth_to_space", x, [r, 0]), crd)
    b, c, h, w = x.shape
    dcr = x.reshape(b, r, r, c // (r * r), h, w).transpose(0, 3, 4, 1, 5, 2).reshape(b, c // (r * r), h * r, w * r)
    assert np.array_equal(O.move_i8("depth_to_space", x, [r, 1]), dcr)


@pytest.mark.parametrize("cfg", [
    # n, ic, ih, iw, oc, k, stride, pads(t,b,l,r), dil, groups, output_padding
    (2, 6, 5, 4, 8, 3, (2, 2), (1, 1, 1, 1), (1, 1), 1, (1, 1)),
    (1, 4, 7, 6, 6, 4, (2, 3), (1, 1, 2, 2), (1, 1), 2, (0, 1)),
    (2, 5, 4, 4, 5, 3, (1, 1), (0, 0, 0, 0), (2, 2), 5, (0, 0)),
    (1, 3, 6, 5, 7, 2, (2, 2), (0, 0, 0, 0), (1, 1), 1, (0, 0)),
])
def test_deconv_accumulators_equal_torch_conv_transpose(cfg):
    n, ic, ih, iw, oc, k, stride, pads, dil, g, opad = cfg
    rng = np.random.default_rng(ic + oc)
    x = rng.integers(-128, 128, (n, ic, ih, iw)).astype(np.int8)
    w = rng.integers(-127, 128, (oc, ic // g, k, k)).astype(np.int8)       # oihw / goihw
    # torch wants (ic, oc // g, kh, kw)
    wt = w.reshape(g, oc // g, ic // g, k, k).transpose(0, 2, 1, 3, 4).reshape(ic, oc // g, k, k)
    want = torch.nn.functional.conv_transpose2d(
        torch.from_numpy(x.astype(np.float64)), torch.from_numpy(wt.astype(np.float64)), None, stride,
        (pads[0], pads[2]), opad, g, dil).numpy()
    d = O.make_deconv_desc(x.shape, w.shape, g, stride, pads, dil, want.shape[2:])
    assert np.array_equal(O.deconv2d_acc(x, w, d), want.astype(np.int64))


def test_bf16_rounding_is_round_to_nearest_even_like_torch():
    rng = np.random.default_rng(11)
    vals = np.concatenate([rng.normal(0, 50, 4000), rng.normal(0, 1e-3, 500), [0.0, 1.0, -1.0, 3.140625,
                           1.00390625, 1.01171875, 255.5, -255.5, 65504.0]]).astype(np.float32)
    want = torch.from_numpy(vals).to(torch.bfloat16).to(torch.float32).numpy()
    got = np.array([O.lib.orc_bf16(float(v), 1) for v in vals], np.float32)
    assert np.array_equal(got, want)
    # truncation mode keeps the high 16 bits
    assert O.lib.orc_bf16(1.01171875, 0) == 1.0078125


def test_quantize_rounds_half_away_from_zero_and_saturates():
    from fractions import Fraction
    rng = np.random.default_rng(12)
    x = np.concatenate([rng.normal(0, 2, 3000), [0.5, -0.5, 1.5, -1.5, 2.5, 126.5, 127.49, 127.5, -128.5,
                        -129.0, 1e6, -1e6, 0.0]]).astype(np.float32)
    for scale in (1.0, 0.37, 63.5, 127.0 / 2.64):
        got = O.quant_f32_to_i8(x, scale)
        prod = x * np.float32(scale)                       # the float32 product the reference forms
        for v, g in zip(prod, got):
            f = Fraction(float(v))
            r = int(abs(f) + Fraction(1, 2))               # nearest, ties away from zero
            r = r if f >= 0 else -r
            assert g == max(-128, min(127, r)), (float(v), scale)


def test_dequantize_is_bf16_of_value_times_bf16_scale():
    x = np.arange(-128, 128, dtype=np.int8)
    for scale in (1.0, 0.0207, 2.64 / 127.0, 3.7):
        s = torch.tensor(scale, dtype=torch.float32).to(torch.bfloat16).to(torch.float32)
        want = (torch.from_numpy(x.astype(np.float32)) * s).to(torch.bfloat16).to(torch.float32).numpy()
        assert np.array_equal(O.dequant_i8_to_f32(x, scale), want)
