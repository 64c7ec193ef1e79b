"""GPU parity tests of the depthwise -> pointwise chain (tpuhip_conv2d_chain_* with a depthwise first
conv): depthwise conv A, an optional 256-entry table on its result, pointwise conv B, an optional
EltwiseAdd on B's result -- every tensor equal to the oracle's ops run one after the other."""
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


def rnd_params(rng, oc, rs_lo=6, rs_hi=14, bias_mag=2048):
    bias = rng.integers(-bias_mag, bias_mag + 1, oc).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
    rsh = rng.integers(rs_lo, rs_hi + 1, oc).astype(np.float32)
    return bias, rsh, mult


def oracle_conv(x, w, p, g, stride, pads, dil, relu):
    d = O.make_conv_desc(x.shape, w.shape, g, stride, pads, dil, (0, 0), relu, True, None)
    return O.conv2d_i8(x, w, p[0], p[1], p[2], d)


def run_dwpw(ctx, rng, c, oc, nhw, k=(3, 3), stride=(1, 1), pads=(1, 1, 1, 1), dil=(1, 1), relu_a=True, relu_b=False,
             table=None, add=None, keep_a=True, keep_lut=True, keep_b=True, rs_lo=6, rs_hi=14):
    n, h, w = nhw
    x = rnd_i8(rng, (n, c, h, w))
    wa, wb = rnd_w(rng, (c, 1) + tuple(k), 40), rnd_w(rng, (oc, c, 1, 1), 12)
    pa, pb = rnd_params(rng, c, rs_lo, rs_hi), rnd_params(rng, oc, rs_lo + 2, rs_hi + 2)
    ya = oracle_conv(x, wa, pa, c, stride, pads, dil, relu_a)
    mid = ya
    if table is not None:
        mid = table[ya.view(np.uint8)]
    yb = oracle_conv(mid, wb, pb, 1, (1, 1), (0, 0, 0, 0), (1, 1), relu_b)
    total = yb
    if add:
        other = rnd_i8(rng, yb.shape)
        m_src, m_conv, rs, relu = add
        total = O.eltwise_add_i8([other, yb], [m_src, m_conv], [rs], relu)
    da = conv_desc(x.shape, wa.shape, g=c, stride=stride, pads=pads, dil=dil, do_relu=relu_a)
    db = conv_desc(ya.shape, wb.shape, do_relu=relu_b)
    assert ctx.conv_chain_kind(da, db) == 2
    ch = ctx.conv_chain_prepack(da, db, (wa, f2i32(pa[0]), f2i32(pa[2]), f2i32(pa[1])),
                                (wb, f2i32(pb[0]), f2i32(pb[2]), f2i32(pb[1])))
    assert ctx.conv_chain_name(ch).startswith("mfma_dwpw_")
    xt = ctx.from_nchw(x)
    yat, lt, ybt, zt = ctx.tensor(ya.shape), ctx.tensor(ya.shape), ctx.tensor(yb.shape), ctx.tensor(yb.shape)
    for t in (yat, lt, ybt, zt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    ot = ctx.from_nchw(other) if add else None
    ctx.conv_chain_post(ch, xt, y_b=ybt if keep_b else None, y_a=yat if keep_a else None, table_a=table,
                        lut_out_a=lt if (table is not None and keep_lut) else None,
                        add_b=(ot, zt, *add) if add else None)
    if keep_b:
        assert np.array_equal(ctx.to_nchw(ybt), yb), "conv B"
        assert not ctx.raw(ybt)[..., oc:].any(), "pad channels of B's result"
    else:
        assert (ctx.raw(ybt) == 0x55).all()
    if keep_a:
        assert np.array_equal(ctx.to_nchw(yat), ya), "conv A"
        assert not ctx.raw(yat)[..., c:].any(), "pad channels of A's result"
    else:
        assert (ctx.raw(yat) == 0x55).all()
    if table is not None and keep_lut:
        assert np.array_equal(ctx.to_nchw(lt), mid), "table"
        assert not ctx.raw(lt)[..., c:].any(), "pad channels of the table's result"
    else:
        assert (ctx.raw(lt) == 0x55).all()
    if add:
        assert np.array_equal(ctx.to_nchw(zt), total), "sum"
    else:
        assert (ctx.raw(zt) == 0x55).all()
    ctx.conv_chain_destroy(ch)
    for t in (xt, yat, lt, ybt, zt) + ((ot,) if ot else ()):
        t.free()


# (depthwise channels, pointwise output channels): the inverted-residual blocks of MobileNetV2 and two
# that are no multiples of 16 or 32
CHANNELS = [(32, 16), (96, 24), (144, 32), (192, 64), (384, 96), (576, 160), (960, 320), (40, 20), (72, 33)]
# (n, h, w): maps narrower and wider than a row segment, odd sizes, several images
MAPS = [(1, 7, 7), (2, 14, 14), (3, 9, 37), (1, 33, 5)]


@pytest.mark.parametrize("chans", CHANNELS)
@pytest.mark.parametrize("nhw", MAPS)
def test_stride_1(ctx, chans, nhw):
    """3x3 / stride 1 / pad 1 depthwise + ReLU, linear projection, residual add -- the middle blocks"""
    rng = np.random.default_rng(chans[0] * 5 + nhw[1])
    run_dwpw(ctx, rng, *chans, nhw, add=(64, 64, 7, False), keep_a=False, keep_b=False)


@pytest.mark.parametrize("chans", CHANNELS[:7:2] + CHANNELS[7:])
@pytest.mark.parametrize("nhw", [(2, 14, 14), (1, 15, 29)])
@pytest.mark.parametrize("pads", [(1, 1, 1, 1), (0, 1, 0, 1)])
def test_stride_2(ctx, chans, nhw, pads):
    """3x3 / stride 2 depthwise (every tap loaded), projection, every tensor kept"""
    rng = np.random.default_rng(chans[0] * 3 + nhw[2] + pads[0])
    run_dwpw(ctx, rng, *chans, nhw, stride=(2, 2), pads=pads)


@pytest.mark.parametrize("k,stride,pads,dil", [
    ((3, 3), (1, 1), (2, 2, 2, 2), (2, 2)),     # dilated
    ((1, 3), (1, 1), (0, 0, 1, 1), (1, 1)),     # one filter row
    ((3, 1), (1, 1), (1, 1, 0, 0), (1, 1)),     # one filter column
    ((2, 2), (2, 2), (0, 0, 0, 0), (1, 1)),
    ((3, 3), (1, 2), (1, 1, 1, 1), (1, 1)),     # stride along W only
    ((3, 3), (2, 1), (1, 1, 1, 1), (1, 1)),     # stride along H only: the neighbour-lane form
    ((1, 1), (1, 1), (0, 0, 0, 0), (1, 1)),
])
def test_windows(ctx, k, stride, pads, dil):
    rng = np.random.default_rng(k[0] * 10 + k[1] + stride[0] + dil[0])
    run_dwpw(ctx, rng, 96, 24, (2, 12, 19), k=k, stride=stride, pads=pads, dil=dil)


@pytest.mark.parametrize("chans", [(96, 24), (384, 64)])
@pytest.mark.parametrize("relu_a,relu_b,table,add,keep_a,keep_lut,keep_b", [
    (True, True, "clip", None, True, True, True),            # ReLU6 as a clip table behind the depthwise conv
    (True, False, "clip", (100, -128, 9, True), False, False, True),   # a shift beyond the packed-int16 add
    (False, False, "any", (-61, 47, 0, False), True, False, False),    # no ReLU anywhere, an arbitrary table
    (False, True, None, None, False, False, True),
    (True, False, None, (61, 47, 6, True), True, False, True),
])
def test_forms(ctx, chans, relu_a, relu_b, table, add, keep_a, keep_lut, keep_b):
    rng = np.random.default_rng(chans[0] + (3 if table else 1) + (7 if add else 0))
    t = None
    if table == "clip":
        t = np.clip(np.arange(256).astype(np.uint8).view(np.int8), 0, 93).astype(np.int8)
    elif table == "any":
        t = rnd_i8(rng, (256,))
    run_dwpw(ctx, rng, *chans, (2, 11, 13), relu_a=relu_a, relu_b=relu_b, table=t, add=add, keep_a=keep_a,
             keep_lut=keep_lut, keep_b=keep_b)


def test_extreme_shifts(ctx):
    rng = np.random.default_rng(11)
    run_dwpw(ctx, rng, 96, 24, (1, 9, 9), relu_a=False, rs_lo=1, rs_hi=29)


def test_many_images_at_full_width(ctx):
    """a MobileNetV2 block at its real shape: 144 channels at 56 x 56, 8 images"""
    rng = np.random.default_rng(12)
    run_dwpw(ctx, rng, 144, 24, (8, 56, 56), add=(64, 64, 7, False), keep_a=False)


def test_refusals(ctx):
    rng = np.random.default_rng(13)
    x = (1, 96, 8, 8)
    da = conv_desc(x, (96, 1, 3, 3), g=96, pads=(1, 1, 1, 1), do_relu=True)
    db = conv_desc(x, (24, 96, 1, 1))
    assert ctx.conv_chain_kind(da, db) == 2
    # a 5x5 depthwise window, a second conv that is no 1x1, one that reads other channels, too many outputs
    assert ctx.conv_chain_kind(conv_desc(x, (96, 1, 5, 5), g=96, pads=(2, 2, 2, 2)), db) == 0
    assert ctx.conv_chain_kind(da, conv_desc(x, (24, 96, 3, 3), pads=(1, 1, 1, 1))) == 0
    assert ctx.conv_chain_kind(da, conv_desc((1, 64, 8, 8), (24, 64, 1, 1))) == 0
    assert ctx.conv_chain_kind(da, conv_desc(x, (400, 96, 1, 1))) == 0
    wa, wb = rnd_w(rng, (96, 1, 3, 3)), rnd_w(rng, (24, 96, 1, 1))
    pa, pb = rnd_params(rng, 96), rnd_params(rng, 24)
    pa[1][5] = 0      # a right shift of 0: the overflow-free rounding needs at least 1
    with pytest.raises(capi.TpuHipError):
        ctx.conv_chain_prepack(da, db, (wa, f2i32(pa[0]), f2i32(pa[2]), f2i32(pa[1])),
                               (wb, f2i32(pb[0]), f2i32(pb[2]), f2i32(pb[1])))
    pa[1][5] = 7
    ch = ctx.conv_chain_prepack(da, db, (wa, f2i32(pa[0]), f2i32(pa[2]), f2i32(pa[1])),
                                (wb, f2i32(pb[0]), f2i32(pb[2]), f2i32(pb[1])))
    xt, yt, zt = ctx.tensor(x), ctx.tensor((1, 24, 8, 8)), ctx.tensor((1, 24, 8, 8))
    with pytest.raises(capi.TpuHipError, match="behind the second conv"):
        ctx.conv_chain(ch, xt, yt, add=(zt, zt, 1, 1, 1, False))     # the pointwise pair's form of the add
    with pytest.raises(capi.TpuHipError, match="no add behind the first"):
        ctx.conv_chain_post(ch, xt, y_b=yt, add_a=(xt, None, 1, 1, 1, False))
    ctx.conv_chain_destroy(ch)
