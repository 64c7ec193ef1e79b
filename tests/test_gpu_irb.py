"""GPU parity tests of the inverted-residual chain (tpuhip_conv2d_chain3_*): 1x1 expansion, depthwise conv,
1x1 projection and the block's EltwiseAdd as one launch -- the result equal to the oracle's ops run one
after the other."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_helpers import conv_desc, f2i32
from tpu_compiler_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def rnd_i8(rng, shape, lo=-128, hi=127):
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int64).astype(np.int8)


def rnd_w(rng, shape, sigma=32):
    return np.clip(np.rint(rng.normal(0, sigma, shape)), -127, 127).astype(np.int8)


def rnd_params(rng, oc, acc_rms=None, rs_lo=6, rs_hi=14, bias_mag=2048):
    """acc_rms: the accumulators' expected magnitude -- shifts are then chosen so that the results keep a
    spread of about 30 and the next layer still has something to work on"""
    bias = rng.integers(-bias_mag, bias_mag + 1, oc).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
    if acc_rms is not None:
        r0 = int(np.clip(round(np.log2(max(acc_rms, 1.0) * 0.75 / 30.0)), 2, 29))
        rs_lo, rs_hi = r0 - 1, r0 + 1
    rsh = rng.integers(rs_lo, rs_hi + 1, oc).astype(np.float32)
    return bias, rsh, mult


def oracle_conv(x, w, p, g, stride, pads, dil, relu):
    d = O.make_conv_desc(x.shape, w.shape, g, stride, pads, dil, (0, 0), relu, True, None)
    return O.conv2d_i8(x, w, p[0], p[1], p[2], d)


def ints(p):
    return f2i32(p[0]), f2i32(p[2]), f2i32(p[1])


def run_irb(ctx, rng, cin, cexp, cout, nhw, k=(3, 3), stride=(1, 1), pads=(1, 1, 1, 1), dil=(1, 1),
            relu=(True, True, False), add=None, keep_y=True, rs_lo=None, rs_hi=None):
    n, h, w = nhw
    x = rnd_i8(rng, (n, cin, h, w))
    we, wd, wp = rnd_w(rng, (cexp, cin, 1, 1), 24), rnd_w(rng, (cexp, 1) + tuple(k), 40), rnd_w(rng, (cout, cexp, 1, 1), 12)
    if rs_lo is None:
        taps = k[0] * k[1]
        pe = rnd_params(rng, cexp, np.sqrt(cin) * 24 * 74)
        pd = rnd_params(rng, cexp, np.sqrt(taps) * 40 * 25)
        pp = rnd_params(rng, cout, np.sqrt(cexp) * 12 * 25)
    else:
        pe, pd, pp = (rnd_params(rng, cexp, None, rs_lo, rs_hi), rnd_params(rng, cexp, None, rs_lo, rs_hi),
                      rnd_params(rng, cout, None, rs_lo, rs_hi))
    ye = oracle_conv(x, we, pe, 1, (1, 1), (0, 0, 0, 0), (1, 1), relu[0])
    yd = oracle_conv(ye, wd, pd, cexp, stride, pads, dil, relu[1])
    yp = oracle_conv(yd, wp, pp, 1, (1, 1), (0, 0, 0, 0), (1, 1), relu[2])
    assert rs_lo is not None or (len(np.unique(yd)) > 8 and len(np.unique(yp)) > 8)
    total = yp
    if add:
        other = rnd_i8(rng, yp.shape)
        m_src, m_conv, rs, arelu = add
        total = O.eltwise_add_i8([other, yp], [m_src, m_conv], [rs], arelu)
    de = conv_desc(x.shape, we.shape, do_relu=relu[0])
    dd = conv_desc(ye.shape, wd.shape, g=cexp, stride=stride, pads=pads, dil=dil, do_relu=relu[1])
    dp = conv_desc(yd.shape, wp.shape, do_relu=relu[2])
    assert ctx.conv_can_chain3(de, dd, dp)
    ch = ctx.conv_chain3_prepack(de, dd, dp, (we, *ints(pe)), (wd, *ints(pd)), (wp, *ints(pp)))
    assert ctx.conv_chain_name(ch).startswith("mfma_irb_")
    xt = ctx.from_nchw(x)
    yt, zt = ctx.tensor(yp.shape), ctx.tensor(yp.shape)
    for t in (yt, zt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    ot = ctx.from_nchw(other) if add else None
    ctx.conv_chain3(ch, xt, yt if keep_y else None, (ot, zt, *add) if add else None)
    if keep_y:
        got = ctx.to_nchw(yt)
        assert np.array_equal(got, yp), "projection: %d mismatches" % (got != yp).sum()
        assert not ctx.raw(yt)[..., cout:].any(), "pad channels of the projection's result"
    else:
        assert (ctx.raw(yt) == 0x55).all()
    if add:
        got = ctx.to_nchw(zt)
        assert np.array_equal(got, total), "sum: %d mismatches" % (got != total).sum()
    else:
        assert (ctx.raw(zt) == 0x55).all()
    ctx.conv_chain_destroy(ch)
    for t in (xt, yt, zt) + ((ot,) if ot else ()):
        t.free()


# (input, expanded, output channels): MobileNetV2's blocks and two that are no multiples of 16 or 32
CHANNELS = [(16, 96, 24), (24, 144, 24), (32, 192, 32), (64, 384, 64), (96, 576, 96), (160, 960, 160), (160, 960, 320),
            (20, 72, 33), (8, 40, 12)]
MAPS = [(1, 7, 7), (2, 14, 14), (3, 9, 37), (1, 33, 5), (2, 28, 28)]


@pytest.mark.parametrize("chans", CHANNELS)
@pytest.mark.parametrize("nhw", MAPS)
def test_stride_1_with_the_residual_add(ctx, chans, nhw):
    rng = np.random.default_rng(chans[1] * 5 + nhw[1])
    same = chans[0] == chans[2]
    run_irb(ctx, rng, *chans, nhw, add=(64, 64, 7, False) if same else None, keep_y=not same)


@pytest.mark.parametrize("chans", [(16, 96, 24), (24, 144, 32), (32, 192, 64), (96, 576, 160), (20, 72, 33)])
@pytest.mark.parametrize("nhw", [(2, 14, 14), (1, 15, 29), (2, 28, 28)])
@pytest.mark.parametrize("pads", [(1, 1, 1, 1), (0, 1, 0, 1)])
def test_stride_2(ctx, chans, nhw, pads):
    rng = np.random.default_rng(chans[1] * 3 + nhw[2] + pads[0])
    run_irb(ctx, rng, *chans, nhw, stride=(2, 2), pads=pads)


@pytest.mark.parametrize("k,stride,pads,dil", [
    ((3, 3), (1, 1), (2, 2, 2, 2), (2, 2)),
    ((1, 3), (1, 1), (0, 0, 1, 1), (1, 1)),
    ((3, 1), (1, 1), (1, 1, 0, 0), (1, 1)),
    ((2, 2), (2, 2), (0, 0, 0, 0), (1, 1)),
    ((3, 3), (1, 2), (1, 1, 1, 1), (1, 1)),
    ((3, 3), (2, 1), (1, 1, 1, 1), (1, 1)),
])
def test_windows(ctx, k, stride, pads, dil):
    rng = np.random.default_rng(k[0] * 10 + k[1] + stride[0] + dil[0])
    run_irb(ctx, rng, 24, 144, 32, (2, 12, 19), k=k, stride=stride, pads=pads, dil=dil)


@pytest.mark.parametrize("relu,add,keep_y", [
    ((True, True, True), None, True),
    ((False, False, False), (-61, 47, 0, False), True),     # no ReLU anywhere: the expansion's padding still is zero
    ((True, False, False), (100, -128, 9, True), False),    # a shift beyond the packed-int16 add
    ((False, True, True), (61, 47, 6, True), False),
])
def test_forms(ctx, relu, add, keep_y):
    rng = np.random.default_rng(sum(relu) * 3 + (7 if add else 0))
    run_irb(ctx, rng, 32, 192, 32, (2, 11, 13), relu=relu, add=add, keep_y=keep_y)


def test_extreme_shifts(ctx):
    rng = np.random.default_rng(11)
    run_irb(ctx, rng, 16, 96, 24, (1, 9, 9), relu=(False, False, False), rs_lo=1, rs_hi=29)


def test_a_block_at_its_real_shape(ctx):
    """MobileNetV2's 14 x 14 blocks at 16 images"""
    rng = np.random.default_rng(12)
    run_irb(ctx, rng, 64, 384, 64, (16, 14, 14), add=(64, 64, 7, False), keep_y=False)


def test_refusals(ctx):
    x = (1, 24, 8, 8)
    de = conv_desc(x, (144, 24, 1, 1), do_relu=True)
    dd = conv_desc((1, 144, 8, 8), (144, 1, 3, 3), g=144, pads=(1, 1, 1, 1), do_relu=True)
    dp = conv_desc((1, 144, 8, 8), (24, 144, 1, 1))
    assert ctx.conv_can_chain3(de, dd, dp)
    # an expansion of too many input channels, a 3x3 first conv, a dense middle conv, a 5x5 window
    assert not ctx.conv_can_chain3(conv_desc((1, 192, 8, 8), (144, 192, 1, 1)), dd, dp)
    assert not ctx.conv_can_chain3(conv_desc(x, (144, 24, 3, 3), pads=(1, 1, 1, 1)), dd, dp)
    assert not ctx.conv_can_chain3(de, conv_desc((1, 144, 8, 8), (144, 144, 3, 3), pads=(1, 1, 1, 1)), dp)
    assert not ctx.conv_can_chain3(de, conv_desc((1, 144, 8, 8), (144, 1, 5, 5), g=144, pads=(2, 2, 2, 2)), dp)
