"""GPU parity tests, op by op, through the C ABI: every result must equal the
oracle's byte for byte (int8 outputs, so the bar is exact equality)."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_helpers import conv_desc, f2i32, pool_desc, run_conv
from tpu_compiler_amd import capi

pytestmark = pytest.mark.gpu


def capi_tile_name(t):
    name = capi.bind().tpuhip_conv2d_tile_name(t)
    return name.decode() if name else None


NUM_TILES = next(t for t in range(1024) if capi_tile_name(t) is None)
# the patch variants take 3x3 / stride 1 / pad 1 layers only; the others take any dense conv
PATCH_TILES = [t for t in range(NUM_TILES) if "mfma_patch_" in capi_tile_name(t)]
# their second form: the same layers, only with the overflow-free requantisation
PATCH2_TILES = [t for t in range(NUM_TILES) if "mfma_patch2_" in capi_tile_name(t)]
# the pointwise variants take unpadded 1x1 layers with at most the K in their name
PW_TILES = [t for t in range(NUM_TILES) if "_pw_" in capi_tile_name(t)]
# their third form: the same layers again; the four waves of a pixel group split K
PATCH3_TILES = [t for t in range(NUM_TILES) if "mfma_patch3_" in capi_tile_name(t)]
GENERAL_TILES = [t for t in range(NUM_TILES) if t not in PATCH_TILES + PATCH2_TILES + PATCH3_TILES + PW_TILES]


def tile_bn(tile):
    """pixel slots of a tile variant named ..._<BM>x<BN>..."""
    return int(capi_tile_name(tile).split("_")[2].split("x")[1])


def tile_k(tile):
    """K bytes a patch variant consumes per step / a pointwise variant holds"""
    name = capi_tile_name(tile)
    return 256 if "k256" in name else 128 if "k128" in name else 64


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def rnd_i8(rng, shape, lo=-128, hi=127):
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int64).astype(np.int8)


def rnd_w(rng, shape, sigma=32):
    return np.clip(np.rint(rng.normal(0, sigma, shape)), -127, 127).astype(np.int8)


def rnd_params(rng, oc, rs_lo=8, rs_hi=20, bias_mag=4096):
    bias = rng.integers(-bias_mag, bias_mag + 1, oc).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
    rsh = rng.integers(rs_lo, rs_hi + 1, oc).astype(np.float32)
    return bias, rsh, mult


def oracle_conv(x, w, bias, rsh, mult, g=1, stride=(1, 1), pads=(0, 0, 0, 0), dil=(1, 1),
                ins=(0, 0), do_relu=False, with_bias=True, out_hw=None):
    d = O.make_conv_desc(x.shape, w.shape, g, stride, pads, dil, ins, do_relu, with_bias, out_hw)
    return O.conv2d_i8(x, w, bias, rsh, mult, d)


# n, ic, ih, iw, oc, kh, kw, stride, pads, dil, relu  (dense convolutions, g = 1)
DENSE = [
    (1, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True),      # config 1
    (2, 64, 14, 14, 256, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), False),    # 1x1, tile 128x128
    (2, 256, 14, 14, 64, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), True),     # tile 64x256
    (1, 3, 32, 32, 64, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1), True),       # stem: 3 channels, 7x7 s2
    (3, 24, 9, 11, 144, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), False),     # ic, oc not multiples of 16/64
    (1, 144, 9, 11, 24, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), False),     # oc 24 -> tile 32x256
    (2, 32, 13, 13, 16, 3, 3, (2, 2), (0, 1, 0, 1), (1, 1), True),      # asymmetric pads, s2
    (1, 48, 10, 10, 80, 3, 3, (1, 1), (2, 2, 2, 2), (2, 2), True),      # dilation 2
    (2, 128, 7, 7, 255, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), False),     # 255 output channels
    (1, 512, 5, 5, 128, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True),      # K = 4608
    (2, 64, 8, 8, 64, 1, 1, (2, 2), (0, 0, 0, 0), (1, 1), False),       # 1x1 stride 2 (downsample)
    (1, 16, 6, 5, 32, 5, 3, (1, 2), (2, 2, 1, 1), (1, 1), False),       # non-square kernel
]


@pytest.mark.parametrize("case", DENSE)
@pytest.mark.parametrize("algo", [capi.ALGO_MFMA, capi.ALGO_DIRECT])
def test_conv_dense(ctx, case, algo):
    n, ic, ih, iw, oc, kh, kw, stride, pads, dil, relu = case
    rng = np.random.default_rng(ic * 1000 + oc + kh)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, kh, kw))
    bias, rsh, mult = rnd_params(rng, oc)
    want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, dil, (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=algo, stride=stride, pads=pads, dil=dil,
                         do_relu=relu)
    assert got.shape == want.shape
    assert np.array_equal(got, want), "%s: %d mismatches" % (name, (got != want).sum())
    # outputs must not be degenerate, or equality proves little
    assert len(np.unique(want)) > 8


# n, ic, ih, iw, oc, kh, kw, stride, pads, relu: at most 4 input channels, at most 64 output channels
STEM_CASES = [
    (2, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3, 3, 3), True),        # ResNet-50 conv1 at a smaller size
    (3, 3, 40, 300, 32, 3, 3, (2, 2), (1, 1, 1, 1), True),       # 150 pixels per row: two segments
    (2, 3, 19, 141, 32, 3, 3, (1, 1), (1, 1, 1, 1), False),      # stride 1, ragged second segment
    (70, 3, 9, 12, 24, 3, 3, (1, 1), (1, 1, 1, 1), True),        # many tiny tiles: the workgroups walk
    (1, 1, 30, 31, 16, 5, 5, (1, 2), (2, 2, 2, 2), False),       # one channel, mixed strides
    (2, 4, 12, 20, 48, 2, 8, (1, 1), (0, 1, 3, 4), False),       # four channels, kw = 8, asymmetric pads
    (1, 2, 17, 9, 64, 7, 1, (3, 1), (3, 3, 0, 0), True),         # kw = 1, stride_h 3
    (2, 3, 21, 21, 40, 4, 6, (2, 2), (1, 2, 2, 3), False),       # even kernel sizes, 40 channels
]


@pytest.mark.parametrize("case", STEM_CASES)
@pytest.mark.parametrize("algo", [capi.ALGO_STEM, capi.ALGO_AUTO])
def test_conv_stem(ctx, case, algo):
    n, ic, ih, iw, oc, kh, kw, stride, pads, relu = case
    rng = np.random.default_rng(ic * 131 + oc + kh * 7 + kw)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, kh, kw))
    bias, rsh, mult = rnd_params(rng, oc)
    want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, (1, 1), (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=algo, stride=stride, pads=pads, do_relu=relu)
    assert name == "stem"
    assert np.array_equal(got, want), "%d mismatches" % (got != want).sum()
    assert len(np.unique(want)) > 8


@pytest.mark.parametrize("case", STEM_CASES)
def test_conv_stem_on_an_input_of_one_dword_per_pixel(ctx, case):
    """the same layers with the input at a channel stride of 4 instead of 16 -- at prepack and switched
    over afterwards; bytes 3 of a 3-channel pixel are zero as the layout conversion writes them"""
    n, ic, ih, iw, oc, kh, kw, stride, pads, relu = case
    rng = np.random.default_rng(ic * 131 + oc + kh * 7 + kw + 1)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, kh, kw))
    bias, rsh, mult = rnd_params(rng, oc)
    want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, (1, 1), (0, 0), relu)
    xt = ctx.from_nchw(x, cs=4)
    assert xt.cs == 4 and xt.nbytes == n * ih * iw * 4
    assert not ctx.raw(xt)[..., ic:].any()
    for at_prepack in (True, False):
        d = conv_desc(x.shape, w.shape, stride=stride, pads=pads, do_relu=relu, x_cs=4 if at_prepack else None)
        wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
        assert ctx.conv_algo_name(wh) == "stem"
        if not at_prepack:
            ctx.conv_set_input_stride(wh, 4)
        yt = ctx.tensor(want.shape)
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
        ctx.conv(wh, xt, yt)
        got = ctx.to_nchw(yt)
        assert np.array_equal(got, want), "%d mismatches" % (got != want).sum()
        ctx.conv_weights_destroy(wh)
        yt.free()
    assert np.array_equal(ctx.to_nchw(xt), x)       # and back through the layout conversion
    xt.free()


def test_conv_off_the_stem_path_refuses_a_dword_input(ctx):
    rng = np.random.default_rng(77)
    w = rnd_w(rng, (128, 3, 3, 3))                   # 128 output channels: the general MFMA path
    bias, rsh, mult = rnd_params(rng, 128)
    with pytest.raises(capi.TpuHipError, match="4-byte channel stride"):
        ctx.conv_prepack(conv_desc((1, 3, 16, 16), w.shape, pads=(1, 1, 1, 1), x_cs=4), w, f2i32(bias), f2i32(mult),
                         f2i32(rsh))
    wh = ctx.conv_prepack(conv_desc((1, 3, 16, 16), w.shape, pads=(1, 1, 1, 1)), w, f2i32(bias), f2i32(mult), f2i32(rsh))
    with pytest.raises(capi.TpuHipError, match="only the stem path"):
        ctx.conv_set_input_stride(wh, 4)
    ctx.conv_weights_destroy(wh)
    with pytest.raises(capi.TpuHipError, match="channel stride"):
        ctx.tensor((1, 8, 4, 4), cs=4)               # 8 channels do not fit a dword


# n, ic, ih, iw, oc, kh, kw, conv stride, conv pads, pool pads (t, b, l, r), pool out_hw or None
STEM_POOL_CASES = [
    (2, 3, 224, 224, 64, 7, 7, (2, 2), (3, 3, 3, 3), (0, 1, 0, 1), None),     # ResNet-50 conv1 + pool1 (Caffe ceil mode)
    (3, 3, 64, 80, 64, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1, 1, 1), None),        # the torchvision form: pool padded by 1
    (1, 3, 57, 61, 48, 5, 5, (2, 2), (2, 2, 2, 2), (0, 0, 0, 0), None),        # odd sizes, 48 channels, 5x5
    (5, 1, 33, 47, 64, 7, 3, (2, 1), (3, 3, 1, 1), (1, 0, 0, 1), None),        # one channel, stride_w 1, mixed pool pads
    (2, 4, 30, 36, 40, 4, 8, (1, 2), (1, 2, 3, 4), (0, 1, 1, 0), None),        # four channels, kw = 8, stride_h 1
    (40, 3, 32, 32, 64, 7, 7, (2, 2), (3, 3, 3, 3), (0, 1, 0, 1), None),       # many images: whole maps per workgroup
]


@pytest.mark.parametrize("case", STEM_POOL_CASES)
@pytest.mark.parametrize("store_conv", [False, True])
def test_conv_stem_with_the_max_pool_in_its_launch(ctx, case, store_conv):
    """conv + ReLU + 3x3 / stride 2 max pool as one launch (tpuhip_conv2d_post_i8 with a pool): the
    pooled tensor equals the oracle's pool of the oracle's conv; the conv result is written only on request"""
    n, ic, ih, iw, oc, kh, kw, stride, pads, ppads, pout = case
    rng = np.random.default_rng(n * 7 + ic * 131 + oc + kh * 7 + kw + ih)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, kh, kw))
    bias, rsh, mult = rnd_params(rng, oc)
    rsh = np.maximum(rsh, 1)
    conv_want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, (1, 1), (0, 0), True)
    pool_want = O.pool_max_i8(conv_want, O.make_pool_desc(conv_want.shape, (3, 3), (2, 2), ppads, pout))
    d = conv_desc(x.shape, w.shape, stride=stride, pads=pads, do_relu=True)
    pd = pool_desc(conv_want.shape, (3, 3), (2, 2), ppads, pout)
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    assert ctx.conv_algo_name(wh) == "stem" and ctx.conv_can_fuse_pool(wh, pd)
    xt = ctx.from_nchw(x)
    yt = ctx.tensor(conv_want.shape)
    pt = ctx.tensor(pool_want.shape)
    for t in (yt, pt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    ctx.conv_post(wh, xt, yt if store_conv else None, pool=(pd, pt))
    got = ctx.to_nchw(pt)
    assert np.array_equal(got, pool_want), "%d mismatches" % (got != pool_want).sum()
    if pt.cs != oc:
        assert not ctx.raw(pt)[..., oc:].any(), "pad channels must be zero"
    if store_conv:
        assert np.array_equal(ctx.to_nchw(yt), conv_want)
    else:
        assert (ctx.raw(yt) == 0x55).all(), "the conv result was not asked for"
    assert len(np.unique(pool_want)) > 8
    ctx.conv_weights_destroy(wh)


def test_conv_stem_refuses_pools_it_cannot_take(ctx):
    rng = np.random.default_rng(5)
    shape = (1, 3, 32, 32)
    w = rnd_w(rng, (64, 3, 7, 7))
    bias, rsh, mult = rnd_params(rng, 64)
    rsh = np.maximum(rsh, 1)
    out = (1, 64, 16, 16)
    ok_pool = pool_desc(out, (3, 3), (2, 2), (0, 1, 0, 1))

    def packed(**kw):
        d = conv_desc(shape, w.shape, stride=(2, 2), pads=(3, 3, 3, 3), **kw)
        return ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))

    wh = packed(do_relu=True)
    assert ctx.conv_can_fuse_pool(wh, ok_pool)
    for bad in (pool_desc(out, (2, 2), (2, 2), (0, 0, 0, 0)), pool_desc(out, (3, 3), (1, 1), (1, 1, 1, 1)),
                pool_desc(out, (3, 3), (2, 2), (2, 2, 2, 2)), pool_desc((1, 64, 16, 18), (3, 3), (2, 2), (0, 1, 0, 1))):
        assert not ctx.conv_can_fuse_pool(wh, bad)
    xt, pt = ctx.from_nchw(np.zeros(shape, np.int8)), ctx.tensor((1, 64, 8, 8))
    with pytest.raises(capi.TpuHipError, match="cannot take the max pool"):
        ctx.conv_post(wh, xt, None, pool=(pool_desc(out, (2, 2), (2, 2), (0, 0, 0, 0)), pt))
    ctx.conv_weights_destroy(wh)
    no_relu = packed(do_relu=False)        # the pool stage relies on bytes in 0..127
    assert not ctx.conv_can_fuse_pool(no_relu, ok_pool)
    ctx.conv_weights_destroy(no_relu)


def test_conv_stem_general_requant_fused_table_and_limits(ctx):
    """parameters outside the overflow-free form, a table fused behind the requantisation, and the
    shapes the stem path refuses"""
    rng = np.random.default_rng(991)
    x = rnd_i8(rng, (2, 3, 33, 35))
    w = rnd_w(rng, (32, 3, 3, 3), sigma=60)
    bias = rng.integers(-(1 << 23), 1 << 23, 32).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, 32) * 128).astype(np.float32)
    rsh = rng.integers(0, 9, 32).astype(np.float32)
    rsh[:4] = 0
    want = oracle_conv(x, w, bias, rsh, mult, 1, (1, 1), (1, 1, 1, 1), (1, 1), (0, 0), False)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=capi.ALGO_STEM, pads=(1, 1, 1, 1))
    assert name == "stem" and np.array_equal(got, want)
    table = rng.integers(-128, 128, 256).astype(np.int8)
    table[0] = 77
    d = conv_desc(x.shape, w.shape, pads=(1, 1, 1, 1), algo=capi.ALGO_STEM)
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    xt, yt, tt = ctx.from_nchw(x), ctx.tensor(want.shape), ctx.tensor(want.shape)
    ctx.conv_post(wh, xt, yt, table, tt)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert np.array_equal(ctx.to_nchw(tt), O.lut_i8(want, table))
    ctx.conv_weights_destroy(wh)
    for shape, wshape, kw_ in [((1, 8, 9, 9), (16, 8, 3, 3), {}), ((1, 3, 9, 9), (80, 3, 3, 3), {}),
                               ((1, 3, 9, 9), (16, 3, 3, 3), dict(dil=(2, 2))),
                               ((1, 3, 30, 30), (16, 3, 3, 3), dict(stride=(1, 3)))]:
        dd = conv_desc(shape, wshape, algo=capi.ALGO_STEM, **kw_)
        ww = np.zeros(wshape, np.int8)
        z = np.zeros(wshape[0], np.int32)
        with pytest.raises(capi.TpuHipError, match="stem path needs"):
            ctx.conv_prepack(dd, ww, z, z + (1 << 30), z + 1)


# n, ic, ih, iw, oc_a, oc_b, k, stride, pads, relu_a, relu_b, bias_b
PAIR_CASES = [
    (2, 64, 14, 14, 256, 64, 1, (1, 1), (0, 0, 0, 0), False, True, True),     # shortcut + first 1x1 of a block
    (3, 256, 15, 13, 512, 128, 1, (2, 2), (0, 0, 0, 0), False, True, True),   # the strided pair
    (1, 40, 9, 11, 128, 24, 3, (1, 1), (1, 1, 1, 1), True, False, False),     # ragged second half, 3x3
    (16, 32, 28, 28, 128, 40, 1, (1, 1), (0, 0, 0, 0), True, True, True),     # enough pixels to walk tiles
]


@pytest.mark.parametrize("case", PAIR_CASES)
def test_conv_pair_equals_two_convs(ctx, case):
    n, ic, ih, iw, oca, ocb, k, stride, pads, relu_a, relu_b, bias_b = case
    rng = np.random.default_rng(oca * 7 + ocb + ic)
    x = rnd_i8(rng, (n, ic, ih, iw))
    wa, wb = rnd_w(rng, (oca, ic, k, k)), rnd_w(rng, (ocb, ic, k, k))
    ba, ra, ma = rnd_params(rng, oca)
    bb, rb, mb = rnd_params(rng, ocb, 6, 14)
    want_a = oracle_conv(x, wa, ba, ra, ma, 1, stride, pads, (1, 1), (0, 0), relu_a)
    want_b = oracle_conv(x, wb, bb if bias_b else np.zeros_like(bb), rb, mb, 1, stride, pads, (1, 1), (0, 0), relu_b)
    da = conv_desc(x.shape, wa.shape, stride=stride, pads=pads, do_relu=relu_a)
    db = conv_desc(x.shape, wb.shape, stride=stride, pads=pads, do_relu=relu_b, with_bias=bias_b)
    wh = ctx.conv_prepack_pair(da, db, (wa, f2i32(ba), f2i32(ma), f2i32(ra)),
                               (wb, f2i32(bb) if bias_b else None, f2i32(mb), f2i32(rb)))
    xt, ya, yb = ctx.from_nchw(x), ctx.tensor(want_a.shape), ctx.tensor(want_b.shape)
    for t in (ya, yb):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))      # poison: pads must be rewritten
    ctx.conv_pair(wh, xt, ya, yb)
    assert ctx.conv_algo_name(wh).startswith("mfma")
    assert np.array_equal(ctx.to_nchw(ya), want_a), "%d mismatches in a" % (ctx.to_nchw(ya) != want_a).sum()
    assert np.array_equal(ctx.to_nchw(yb), want_b), "%d mismatches in b" % (ctx.to_nchw(yb) != want_b).sum()
    assert not ctx.raw(yb)[..., ocb:].any() and not ctx.raw(ya)[..., oca:].any()
    assert len(np.unique(want_a)) > 8 and len(np.unique(want_b)) > 8
    # every tile variant splits its output the same way (a pointwise variant takes the pair if it takes
    # the layer and the first conv ends at one of its tile boundaries)
    ran_pw = 0
    for tile in GENERAL_TILES + PW_TILES:
        da.algo = db.algo = 16 + tile
        try:
            wt = ctx.conv_prepack_pair(da, db, (wa, f2i32(ba), f2i32(ma), f2i32(ra)),
                                       (wb, f2i32(bb) if bias_b else None, f2i32(mb), f2i32(rb)))
        except capi.TpuHipError as e:
            assert tile in PW_TILES and "tile" in str(e), str(e)
            continue
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, ya.ptr, 0x55, ya.nbytes))
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yb.ptr, 0x55, yb.nbytes))
        try:
            ctx.conv_pair(wt, xt, ya, yb)
        except capi.TpuHipError as e:
            assert tile in PW_TILES and "tile variant" in str(e), str(e)
            ctx.conv_weights_destroy(wt)
            continue
        ran_pw += tile in PW_TILES
        name = ctx.conv_algo_name(wt)
        assert np.array_equal(ctx.to_nchw(ya), want_a) and np.array_equal(ctx.to_nchw(yb), want_b), name
        ctx.conv_weights_destroy(wt)
    assert ran_pw >= (1 if k == 1 else 0)
    # a pair handle does not run as a single conv, nor a single conv as a pair
    with pytest.raises(capi.TpuHipError, match="pair"):
        ctx.conv(wh, xt, ya)
    ctx.conv_weights_destroy(wh)


def test_conv_pair_refuses_mismatched_convs(ctx):
    x_shape = (1, 32, 8, 8)
    z = lambda oc: (np.zeros((oc, 32, 1, 1), np.int8), None, np.full(oc, 1 << 30, np.int32), np.ones(oc, np.int32))
    da = conv_desc(x_shape, (128, 32, 1, 1))
    with pytest.raises(capi.TpuHipError, match="same window geometry"):
        ctx.conv_prepack_pair(da, conv_desc(x_shape, (16, 32, 1, 1), stride=(2, 2)), z(128), z(16))
    with pytest.raises(capi.TpuHipError, match="multiple of 128"):
        ctx.conv_prepack_pair(conv_desc(x_shape, (64, 32, 1, 1)), conv_desc(x_shape, (16, 32, 1, 1)), z(64), z(16))
    w = ctx.conv_prepack(da, *[z(128)[i] for i in (0, 1, 2, 3)])
    xt, ya = ctx.tensor(x_shape), ctx.tensor((1, 128, 8, 8))
    with pytest.raises(capi.TpuHipError, match="not packed as a pair"):
        ctx.conv_pair(w, xt, ya, ya)
    ctx.conv_weights_destroy(w)


TILE_CASES = [
    (1, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True),
    (2, 96, 17, 13, 200, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), False),   # ragged pixel / channel tails
    (1, 40, 9, 9, 72, 3, 3, (2, 2), (1, 1, 1, 1), (1, 1), True),
    (3, 16, 5, 5, 16, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), False),      # one K step, tiny
    (1, 256, 6, 6, 300, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True),     # 36 K steps
    (2, 3, 20, 23, 40, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1), True),      # 3 channels: 4-tap K packing
    (1, 4, 11, 9, 24, 3, 3, (1, 1), (1, 1, 1, 1), (2, 1), False),
]


# large enough that a persistent workgroup walks several pixel tiles
WALK_CASES = [
    (32, 64, 56, 56, 64, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), True),
    (13, 24, 67, 61, 80, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), False),    # ragged rows, general K mode
    (6, 3, 150, 131, 32, 5, 5, (2, 2), (2, 2, 2, 2), (1, 1), True),     # 3 channels
]
PERSISTENT_TILES = [t for t in range(64) if (capi_tile_name(t) or "").startswith("mfma_p_")]


@pytest.mark.parametrize("case", WALK_CASES)
@pytest.mark.parametrize("tile", PERSISTENT_TILES)
def test_conv_persistent_tiles_walk(ctx, case, tile):
    n, ic, ih, iw, oc, kh, kw, stride, pads, dil, relu = case
    rng = np.random.default_rng(ic * 11 + oc + tile)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, kh, kw))
    bias, rsh, mult = rnd_params(rng, oc)
    want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, dil, (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=16 + tile, stride=stride, pads=pads,
                         dil=dil, do_relu=relu)
    assert name.startswith("mfma_p_")
    assert np.array_equal(got, want), "%s: %d mismatches" % (name, (got != want).sum())
    rsh0 = rsh.copy()
    rsh0[0] = 0     # the general requant form of the same tile
    want = oracle_conv(x, w, bias, rsh0, mult, 1, stride, pads, dil, (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh0, mult, algo=16 + tile, stride=stride, pads=pads,
                         dil=dil, do_relu=relu)
    assert np.array_equal(got, want), "%s (general requant): %d mismatches" % (name, (got != want).sum())


# n, c, h, w, oc, relu, fused add: 3x3 / stride 1 / pad 1 layers for the kernels that keep the input
# rows of a tile in LDS
PATCH_CASES = [
    (2, 64, 56, 56, 64, True, False),      # ResNet-50 stage 2
    (3, 128, 28, 28, 128, True, True),     # stage 3, with the add fused behind it
    (2, 256, 14, 14, 256, False, False),   # stage 4: the image splits into two tiles of 7 rows
    (1, 512, 7, 7, 72, True, False),       # whole image in one tile, ragged output channels
    (2, 64, 9, 7, 40, False, True),        # tiny map, 63 of 128 pixel slots idle
    (1, 128, 5, 20, 64, True, False),
    (1, 64, 37, 30, 200, True, False),     # rows do not divide into equal tiles; four channel tiles
    (5, 64, 3, 100, 16, False, False),     # wide and short
]


# a variant with K steps of 128 or 256 bytes takes layers whose channel count is a multiple of that
@pytest.mark.parametrize("tile,case", [(t, c) for t in PATCH_TILES for c in PATCH_CASES if c[1] % tile_k(t) == 0])
def test_conv_patch_tile_variants(ctx, case, tile):
    n, c, h, w_, oc, relu, add = case
    rng = np.random.default_rng(c + h * 3 + oc + tile)
    x = rnd_i8(rng, (n, c, h, w_))
    w = rnd_w(rng, (oc, c, 3, 3), sigma=14)
    bias, rsh, mult = rnd_params(rng, oc)
    for general in (False, True):
        r = rsh.copy()
        if general:
            r[::3] = 0      # an rshift of 0 forces the general requant form
        want = oracle_conv(x, w, bias, r, mult, 1, (1, 1), (1, 1, 1, 1), (1, 1), (0, 0), relu)
        d = conv_desc(x.shape, w.shape, pads=(1, 1, 1, 1), do_relu=relu, algo=16 + tile)
        xt, yt = ctx.from_nchw(x), ctx.tensor(want.shape)
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
        wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(r))
        assert "patch" in ctx.conv_algo_name(wh)
        if add:
            other = rnd_i8(rng, want.shape)
            z_ref = O.eltwise_add_i8([other, want], [61, 47], [6], True)
            ot, zt = ctx.from_nchw(other), ctx.tensor(want.shape)
            ctx.conv_add(wh, xt, yt, ot, zt, 61, 47, 6, True)
            assert np.array_equal(ctx.to_nchw(zt), z_ref)
        else:
            ctx.conv(wh, xt, yt)
        got = ctx.to_nchw(yt)
        assert np.array_equal(got, want), "%s: %d mismatches" % (ctx.conv_algo_name(wh), (got != want).sum())
        assert not ctx.raw(yt)[..., oc:].any()
        ctx.conv_weights_destroy(wh)
    assert len(np.unique(want)) > 8


# n, ic, ih, iw, oc, stride, relu: unpadded 1x1 layers for the kernels that keep their filter slice in LDS
PW_CASES = [
    (2, 64, 56, 56, 256, 1, False),     # ResNet-50 stage 2 expansion: whole 256-byte rows per tile
    (2, 256, 56, 56, 64, 1, True),      # its reduction
    (3, 128, 28, 28, 512, 1, False),
    (2, 256, 29, 27, 128, 2, True),     # strided, ragged pixel tail
    (1, 40, 9, 11, 72, 1, True),        # K padded from 48 to 64, ragged channels
    (1, 200, 5, 7, 300, 1, False),      # K padded from 208 to 256
    (6, 96, 31, 17, 100, 1, False),     # K 96 -> 128
    (40, 64, 30, 30, 64, 1, True),      # enough pixels that every workgroup walks several tiles
    (1, 16, 1, 1, 16, 1, False),        # one pixel
]


@pytest.mark.parametrize("tile,case", [(t, c) for t in PW_TILES for c in PW_CASES
                                       if (c[1] + 15) // 16 * 16 <= tile_k(t) and
                                       (tile_k(t) == 64 or (c[1] + 15) // 16 * 16 > tile_k(t) // 2)])
@pytest.mark.parametrize("post", ["plain", "add", "add_only", "table_add"])
def test_conv_pointwise_tile_variants(ctx, case, tile, post):
    n, ic, ih, iw, oc, stride, relu = case
    rng = np.random.default_rng(ic * 13 + oc + tile)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, 1, 1))
    bias, rsh, mult = rnd_params(rng, oc)
    y_ref = oracle_conv(x, w, bias, rsh, mult, 1, (stride, stride), (0, 0, 0, 0), (1, 1), (0, 0), relu)
    d = conv_desc(x.shape, w.shape, stride=(stride, stride), do_relu=relu, algo=16 + tile)
    xt = ctx.from_nchw(x)
    yt, tt, zt = ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape)
    for t in (yt, tt, zt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))      # poison: pads must be rewritten
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    assert "_pw_" in ctx.conv_algo_name(wh)
    other = rnd_i8(rng, y_ref.shape)
    ot = ctx.from_nchw(other)
    if post == "plain":
        ctx.conv(wh, xt, yt)
    elif post in ("add", "add_only"):
        z_ref = O.eltwise_add_i8([other, y_ref], [-61, 47], [6], post == "add")
        ctx.conv_add(wh, xt, yt if post == "add" else None, ot, zt, -61, 47, 6, post == "add")
        assert np.array_equal(ctx.to_nchw(zt), z_ref)
        assert not ctx.raw(zt)[..., oc:].any()
    else:
        table = rnd_i8(rng, 256)
        table[0] = 77                                  # pad channels must stay 0 all the same
        t_ref = O.lut_i8(y_ref, table)
        z_ref = O.eltwise_add_i8([other, t_ref], [37, 51], [5], True)
        ctx.conv_post(wh, xt, yt, table, tt, (ot, zt, 37, 51, 5, True))
        assert np.array_equal(ctx.to_nchw(tt), t_ref) and not ctx.raw(tt)[..., oc:].any()
        assert np.array_equal(ctx.to_nchw(zt), z_ref) and not ctx.raw(zt)[..., oc:].any()
    if post == "add_only":
        assert (ctx.raw(yt) == 0x55).all()      # the conv result was not written
    else:
        got = ctx.to_nchw(yt)
        assert np.array_equal(got, y_ref), "%s: %d mismatches" % (ctx.conv_algo_name(wh), (got != y_ref).sum())
        assert not ctx.raw(yt)[..., oc:].any()
    assert y_ref.size < 1000 or len(np.unique(y_ref)) > 8
    ctx.conv_weights_destroy(wh)
    for t in (xt, ot, yt, tt, zt):
        t.free()


@pytest.mark.parametrize("tile", PW_TILES)
def test_conv_pointwise_tiles_refuse_other_layers(ctx, tile):
    """3x3, padded, too many channels, an rshift of 0 (the general requant form): refused by name"""
    k = tile_k(tile)
    ok = lambda oc: (None, np.full(oc, 1 << 30, np.int32), np.full(oc, 8, np.int32))
    xt, yt = ctx.tensor((1, 2 * k, 8, 8)), ctx.tensor((1, 32, 8, 8))
    for shape, wshape, kw, rs0 in (((1, 64, 8, 8), (32, 64, 3, 3), dict(pads=(1, 1, 1, 1)), False),
                                   ((1, 2 * k, 8, 8), (32, 2 * k, 1, 1), {}, False),
                                   ((1, k, 6, 6), (32, k, 1, 1), dict(pads=(1, 1, 1, 1)), False),
                                   ((1, k, 8, 8), (32, k, 1, 1), {}, True)):
        d = conv_desc(shape, wshape, algo=16 + tile, **kw)
        b, m, r = ok(wshape[0])
        if rs0:
            r = r.copy()
            r[5] = 0
        with pytest.raises(capi.TpuHipError, match="tile"):
            wh = ctx.conv_prepack(d, np.ones(wshape, np.int8), b, m, r)
            try:
                ctx.conv(wh, xt, yt)
            finally:
                ctx.conv_weights_destroy(wh)
    xt.free()
    yt.free()


@pytest.mark.parametrize("tile,case", [(t, c) for t in PATCH2_TILES for c in PATCH_CASES if c[3] <= tile_bn(t)])
@pytest.mark.parametrize("post", ["plain", "add", "table_add"])
def test_conv_patch2_tile_variants(ctx, case, tile, post):
    n, c, h, w_, oc, relu, _ = case
    rng = np.random.default_rng(c + h * 3 + oc + tile)
    x = rnd_i8(rng, (n, c, h, w_))
    w = rnd_w(rng, (oc, c, 3, 3), sigma=14)
    bias, rsh, mult = rnd_params(rng, oc)
    rsh[1::5] = 1                      # the smallest shift the overflow-free form takes
    y_ref = oracle_conv(x, w, bias, rsh, mult, 1, (1, 1), (1, 1, 1, 1), (1, 1), (0, 0), relu)
    d = conv_desc(x.shape, w.shape, pads=(1, 1, 1, 1), do_relu=relu, algo=16 + tile)
    xt = ctx.from_nchw(x)
    yt, tt, zt = ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape)
    for t in (yt, tt, zt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    assert "patch2" in ctx.conv_algo_name(wh)
    other = rnd_i8(rng, y_ref.shape)
    ot = ctx.from_nchw(other)
    if post == "plain":
        ctx.conv(wh, xt, yt)
    elif post == "add":
        z_ref = O.eltwise_add_i8([other, y_ref], [61, -47], [6], True)
        ctx.conv_add(wh, xt, yt, ot, zt, 61, -47, 6, True)
        assert np.array_equal(ctx.to_nchw(zt), z_ref) and not ctx.raw(zt)[..., oc:].any()
    else:
        table = rnd_i8(rng, 256)
        table[0] = 77
        t_ref = O.lut_i8(y_ref, table)
        z_ref = O.eltwise_add_i8([other, t_ref], [37, 51], [5], False)
        ctx.conv_post(wh, xt, yt, table, tt, (ot, zt, 37, 51, 5, False))
        assert np.array_equal(ctx.to_nchw(tt), t_ref) and not ctx.raw(tt)[..., oc:].any()
        assert np.array_equal(ctx.to_nchw(zt), z_ref) and not ctx.raw(zt)[..., oc:].any()
    got = ctx.to_nchw(yt)
    assert np.array_equal(got, y_ref), "%s: %d mismatches" % (ctx.conv_algo_name(wh), (got != y_ref).sum())
    assert not ctx.raw(yt)[..., oc:].any()
    assert len(np.unique(y_ref)) > 8
    ctx.conv_weights_destroy(wh)
    for t in (xt, ot, yt, tt, zt):
        t.free()


# cases of the third form beyond PATCH_CASES: tiles of several whole images (with a last tile
# that holds fewer), 1024 input channels, a K that leaves the four K groups unequal shares
PATCH3_CASES = PATCH_CASES + [
    (5, 512, 7, 7, 40, True, False),       # two or five images per tile, the last tile ragged
    (9, 64, 4, 5, 33, False, False),       # up to twelve images per tile
    (2, 1024, 3, 3, 64, True, False),
    (7, 64, 6, 6, 96, True, False),        # 18 K slices: shares of 5, 5, 4 and 4
    (1, 256, 16, 16, 32, False, False),    # exactly 256 pixels
    (8, 128, 1, 30, 20, False, False),     # images of one row, several per tile (a division by H = 1)
    (9, 64, 1, 1, 40, True, False),        # images of one pixel (a division by H * W = 1)
]


@pytest.mark.parametrize("tile,case", [(t, c) for t in PATCH3_TILES for c in PATCH3_CASES if c[3] <= tile_bn(t)])
@pytest.mark.parametrize("post", ["plain", "add", "table_add"])
def test_conv_patch3_tile_variants(ctx, case, tile, post):
    n, c, h, w_, oc, relu, _ = case
    rng = np.random.default_rng(c + h * 3 + oc + tile)
    x = rnd_i8(rng, (n, c, h, w_))
    w = rnd_w(rng, (oc, c, 3, 3), sigma=14)
    bias, rsh, mult = rnd_params(rng, oc)
    rsh[1::5] = 1                      # the smallest shift the overflow-free form takes
    y_ref = oracle_conv(x, w, bias, rsh, mult, 1, (1, 1), (1, 1, 1, 1), (1, 1), (0, 0), relu)
    d = conv_desc(x.shape, w.shape, pads=(1, 1, 1, 1), do_relu=relu, algo=16 + tile)
    xt = ctx.from_nchw(x)
    yt, tt, zt = ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape)
    for t in (yt, tt, zt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    assert "patch3" in ctx.conv_algo_name(wh)
    other = rnd_i8(rng, y_ref.shape)
    ot = ctx.from_nchw(other)
    if post == "plain":
        ctx.conv(wh, xt, yt)
    elif post == "add":
        z_ref = O.eltwise_add_i8([other, y_ref], [61, -47], [6], True)
        ctx.conv_add(wh, xt, yt, ot, zt, 61, -47, 6, True)
        assert np.array_equal(ctx.to_nchw(zt), z_ref) and not ctx.raw(zt)[..., oc:].any()
    else:
        table = rnd_i8(rng, 256)
        table[0] = 77
        t_ref = O.lut_i8(y_ref, table)
        z_ref = O.eltwise_add_i8([other, t_ref], [37, 51], [5], False)
        ctx.conv_post(wh, xt, yt, table, tt, (ot, zt, 37, 51, 5, False))
        assert np.array_equal(ctx.to_nchw(tt), t_ref) and not ctx.raw(tt)[..., oc:].any()
        assert np.array_equal(ctx.to_nchw(zt), z_ref) and not ctx.raw(zt)[..., oc:].any()
    got = ctx.to_nchw(yt)
    assert np.array_equal(got, y_ref), "%s: %d mismatches" % (ctx.conv_algo_name(wh), (got != y_ref).sum())
    assert not ctx.raw(yt)[..., oc:].any()
    assert len(np.unique(y_ref)) > 8
    ctx.conv_weights_destroy(wh)
    for t in (xt, ot, yt, tt, zt):
        t.free()


@pytest.mark.parametrize("tile", PATCH3_TILES)
def test_conv_patch3_tiles_refuse_other_layers(ctx, tile):
    """stride 2, 96 channels, 1x1, a map wider than the tile, an rshift of 0 (the general requant form)"""
    z = lambda oc, ic, k: (np.zeros((oc, ic, k, k), np.int8), None, np.full(oc, 1 << 30, np.int32), np.ones(oc, np.int32))
    for shape, wshape, kw, rs0 in [((1, 64, 8, 8), (64, 64, 3, 3), dict(stride=(2, 2), pads=(1, 1, 1, 1)), False),
                                   ((1, 96, 8, 8), (64, 96, 3, 3), dict(pads=(1, 1, 1, 1)), False),
                                   ((1, 64, 8, 8), (64, 64, 1, 1), dict(), False),
                                   ((1, 64, 8, 300), (64, 64, 3, 3), dict(pads=(1, 1, 1, 1)), False),
                                   ((1, 64, 8, 8), (64, 64, 3, 3), dict(pads=(1, 1, 1, 1)), True)]:
        d = conv_desc(shape, wshape, algo=16 + tile, **kw)
        wt, b, m, r = z(wshape[0], wshape[1], wshape[2])
        if rs0:
            r = r.copy()
            r[5] = 0
        xt, yt = ctx.tensor(shape), ctx.tensor((d.n, d.oc, d.oh, d.ow))
        with pytest.raises(capi.TpuHipError, match="3x3 / stride 1 / pad 1"):
            wh = ctx.conv_prepack(d, wt, b, m, r)
            try:
                ctx.conv(wh, xt, yt)
            finally:
                ctx.conv_weights_destroy(wh)
        xt.free()
        yt.free()


def _random_conv_case(rng):
    """a dense conv of one of three families: 3x3 / stride 1 / pad 1 on the channel counts the
    row-patch kernels take, 1x1 with stride 1 or 2, or anything goes"""
    kind = int(rng.integers(0, 4))
    if kind == 0:
        ic, kh, kw, stride, pads, dil = int(rng.choice([64, 128, 256, 512])), 3, 3, (1, 1), (1, 1, 1, 1), (1, 1)
        iw, n, oc = int(rng.integers(1, 130)), int(rng.integers(1, 4)), int(rng.integers(1, 200))
        ih = min(int(rng.integers(1, 40)), max(1, 400000 // (n * iw * ic)))
    elif kind == 1:
        s = int(rng.integers(1, 3))
        ic, kh, kw, stride, pads, dil = int(rng.integers(1, 300)), 1, 1, (s, s), (0, 0, 0, 0), (1, 1)
        ih, iw, n, oc = int(rng.integers(1, 30)), int(rng.integers(1, 30)), int(rng.integers(1, 5)), int(rng.integers(1, 400))
    else:
        ic, kh, kw = int(rng.integers(1, 100)), int(rng.integers(1, 6)), int(rng.integers(1, 6))
        stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pads = tuple(int(v) for v in rng.integers(0, 4, 4))
        ih, iw, n, oc = int(rng.integers(1, 24)), int(rng.integers(1, 24)), int(rng.integers(1, 4)), int(rng.integers(1, 150))
        if ih + pads[0] + pads[1] < dil[0] * (kh - 1) + 1 or iw + pads[2] + pads[3] < dil[1] * (kw - 1) + 1:
            return None
    return n, ic, ih, iw, oc, kh, kw, stride, pads, dil


@pytest.mark.parametrize("seed", range(6))
def test_conv_random_shapes_every_tile_variant(ctx, seed):
    """25 random convs per seed, each through every tile variant that takes it, with and without
    the fused add and with both requant forms; all must give the oracle's bytes"""
    ran = set()
    for it in range(25):
        rng = np.random.default_rng(7000 + seed * 100 + it)
        case = _random_conv_case(rng)
        if case is None:
            continue
        n, ic, ih, iw, oc, kh, kw, stride, pads, dil = case
        relu, add, general = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), rng.integers(0, 4) == 0
        x = rnd_i8(rng, (n, ic, ih, iw))
        w = rnd_w(rng, (oc, ic, kh, kw), sigma=max(2.0, min(40.0, 375.0 / (ic * kh * kw) ** 0.5)))
        bias, rsh, mult = rnd_params(rng, oc, 5, 11)
        if general:
            rsh[::3] = 0
        want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, dil, (0, 0), relu)
        other = rnd_i8(rng, want.shape)
        z_ref = O.eltwise_add_i8([other, want], [61, 47], [6], True)
        xt, ot = ctx.from_nchw(x), ctx.from_nchw(other)
        yt, zt = ctx.tensor(want.shape), ctx.tensor(want.shape)
        for tile in GENERAL_TILES + PATCH_TILES + PATCH2_TILES + PATCH3_TILES + PW_TILES:
            d = conv_desc(x.shape, w.shape, stride=stride, pads=pads, dil=dil, do_relu=relu, algo=16 + tile)
            try:
                wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
            except capi.TpuHipError:
                continue       # this variant does not take the layer
            ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
            try:
                if add:
                    ctx.conv_add(wh, xt, yt, ot, zt, 61, 47, 6, True)
                else:
                    ctx.conv(wh, xt, yt)
            except capi.TpuHipError as e:
                assert "tile variant" in str(e), str(e)
                ctx.conv_weights_destroy(wh)
                continue
            label = (it, capi_tile_name(tile), x.shape, w.shape, stride, pads, dil, relu, add, bool(general))
            assert np.array_equal(ctx.to_nchw(yt), want), label
            assert not ctx.raw(yt)[..., oc:].any(), label
            if add:
                assert np.array_equal(ctx.to_nchw(zt), z_ref), label
            ran.add(capi_tile_name(tile))
            ctx.conv_weights_destroy(wh)
        for t in (xt, ot, yt, zt):
            t.free()
    assert len(ran) >= 15, sorted(ran)


@pytest.mark.parametrize("tile", PATCH_TILES)
def test_conv_patch_tiles_refuse_other_layers(ctx, tile):
    z = lambda oc, ic, k: (np.zeros((oc, ic, k, k), np.int8), None, np.full(oc, 1 << 30, np.int32), np.ones(oc, np.int32))
    for shape, wshape, kw in [((1, 64, 8, 8), (64, 64, 3, 3), dict(stride=(2, 2), pads=(1, 1, 1, 1))),
                              ((1, 96, 8, 8), (64, 96, 3, 3), dict(pads=(1, 1, 1, 1))),
                              ((1, 64, 8, 8), (64, 64, 1, 1), dict()),
                              ((1, 64, 8, 300), (64, 64, 3, 3), dict(pads=(1, 1, 1, 1)))]:
        d = conv_desc(shape, wshape, algo=16 + tile, **kw)
        wh = ctx.conv_prepack(d, *z(wshape[0], wshape[1], wshape[2]))
        xt, yt = ctx.tensor(shape), ctx.tensor((d.n, d.oc, d.oh, d.ow))
        with pytest.raises(capi.TpuHipError, match="3x3 / stride 1 / pad 1"):
            ctx.conv(wh, xt, yt)
        ctx.conv_weights_destroy(wh)
    # nor do they run a pair
    da, db = conv_desc((1, 64, 8, 8), (128, 64, 3, 3), pads=(1, 1, 1, 1), algo=16 + tile), \
        conv_desc((1, 64, 8, 8), (16, 64, 3, 3), pads=(1, 1, 1, 1), algo=16 + tile)
    wp = ctx.conv_prepack_pair(da, db, z(128, 64, 3), z(16, 64, 3))
    with pytest.raises(capi.TpuHipError, match="single 3x3"):
        ctx.conv_pair(wp, ctx.tensor((1, 64, 8, 8)), ctx.tensor((1, 128, 8, 8)), ctx.tensor((1, 16, 8, 8)))
    ctx.conv_weights_destroy(wp)


@pytest.mark.parametrize("case", TILE_CASES)
@pytest.mark.parametrize("tile", GENERAL_TILES)
def test_conv_every_mfma_tile_variant(ctx, case, tile):
    n, ic, ih, iw, oc, kh, kw, stride, pads, dil, relu = case
    rng = np.random.default_rng(ic * 7 + oc + tile)
    x = rnd_i8(rng, (n, ic, ih, iw))
    w = rnd_w(rng, (oc, ic, kh, kw))
    bias, rsh, mult = rnd_params(rng, oc)
    want = oracle_conv(x, w, bias, rsh, mult, 1, stride, pads, dil, (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=16 + tile, stride=stride, pads=pads,
                         dil=dil, do_relu=relu)
    assert np.array_equal(got, want), "%s: %d mismatches" % (name, (got != want).sum())
    # the general (non-fast) requant form of the same tile: an rshift of 0 forces it
    rsh2 = rsh.copy()
    rsh2[::3] = 0
    want = oracle_conv(x, w, bias, rsh2, mult, 1, stride, pads, dil, (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh2, mult, algo=16 + tile, stride=stride, pads=pads,
                         dil=dil, do_relu=relu)
    assert np.array_equal(got, want), "%s general: %d mismatches" % (name, (got != want).sum())


def test_conv_auto_picks_mfma_for_dense_and_depthwise_for_dw(ctx):
    rng = np.random.default_rng(1)
    x = rnd_i8(rng, (1, 32, 8, 8))
    w = rnd_w(rng, (32, 32, 3, 3))
    bias, rsh, mult = rnd_params(rng, 32)
    _, name = run_conv(ctx, x, w, bias, rsh, mult, pads=(1, 1, 1, 1))
    assert name.startswith("mfma")
    wd = rnd_w(rng, (32, 1, 3, 3))
    _, name = run_conv(ctx, x, wd, bias, rsh, mult, g=32, pads=(1, 1, 1, 1))
    assert name == "depthwise"
    wg = rnd_w(rng, (32, 8, 3, 3))
    _, name = run_conv(ctx, x, wg, bias, rsh, mult, g=4, pads=(1, 1, 1, 1))
    assert name == "direct"


# n, c, ih, iw, k, stride, pads, relu
DEPTHWISE = [
    (2, 256, 56, 56, 3, (1, 1), (1, 1, 1, 1), True),     # config 2 (smaller batch)
    (2, 96, 15, 15, 3, (2, 2), (0, 1, 0, 1), True),
    (1, 24, 9, 9, 3, (1, 1), (1, 1, 1, 1), False),       # 24 channels: padded group
    (1, 32, 12, 12, 5, (1, 1), (2, 2, 2, 2), False),
    (1, 16, 7, 7, 7, (1, 1), (0, 0, 0, 0), False),       # global depthwise
    (1, 48, 10, 9, 2, (1, 1), (0, 1, 0, 1), True),       # 2x2: a single tap group
    (16, 96, 112, 112, 3, (1, 1), (1, 1, 1, 1), True),   # more pixels than lanes: every lane walks
    (3, 40, 23, 17, 3, (2, 1), (1, 1, 1, 1), False),     # mixed strides, ragged everything
]


@pytest.mark.parametrize("case", DEPTHWISE)
@pytest.mark.parametrize("algo", [capi.ALGO_DEPTHWISE, capi.ALGO_DEPTHWISE_DOT, capi.ALGO_DIRECT])
def test_conv_depthwise(ctx, case, algo):
    n, c, ih, iw, k, stride, pads, relu = case
    rng = np.random.default_rng(c + k)
    x = rnd_i8(rng, (n, c, ih, iw))
    w = rnd_w(rng, (c, 1, k, k), 24)
    bias, rsh, mult = rnd_params(rng, c, 5, 12, 2048)
    want = oracle_conv(x, w, bias, rsh, mult, c, stride, pads, (1, 1), (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=algo, g=c, stride=stride, pads=pads,
                         do_relu=relu)
    assert np.array_equal(got, want), name
    assert len(np.unique(want)) > 8


# the row-segment form of the depthwise kernel (windows of at most 3 x 3 taps, right shifts of
# at least 1): n, c, ih, iw, kh, kw, stride, pads, dil, relu, table
DEPTHWISE_ROWS = [
    (3, 144, 56, 56, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True, True),     # 30 + 26 outputs per row, 4.5 channel blocks
    (2, 64, 28, 28, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), False, False),    # one segment per row
    (5, 96, 14, 14, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True, True),      # two rows per block
    (9, 48, 7, 7, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True, False),       # three rows per block, odd row count
    (2, 32, 33, 61, 3, 3, (1, 1), (0, 0, 0, 0), (1, 1), False, True),     # unpadded, ragged width
    (2, 16, 20, 35, 3, 3, (1, 1), (1, 2, 2, 1), (1, 1), True, False),     # one channel block, uneven padding
    (2, 96, 112, 112, 3, 3, (2, 2), (0, 1, 0, 1), (1, 1), True, True),    # stride 2: nine loads, no halo
    (4, 192, 28, 28, 3, 3, (2, 2), (1, 1, 1, 1), (1, 1), False, False),   # stride 2 onto 14 x 14
    (3, 40, 15, 13, 3, 3, (2, 2), (1, 1, 1, 1), (1, 1), True, False),     # stride 2 onto 8 x 7
    (2, 24, 19, 30, 1, 3, (1, 1), (0, 0, 1, 1), (1, 1), True, True),      # one row of taps
    (2, 24, 30, 19, 3, 1, (1, 1), (1, 1, 0, 0), (1, 1), False, False),    # one column of taps
    (2, 40, 22, 22, 2, 2, (1, 1), (0, 1, 0, 1), (1, 1), True, False),     # 2 x 2
    (2, 56, 25, 25, 3, 3, (1, 1), (2, 2, 2, 2), (2, 2), True, True),      # dilated both ways
    (2, 56, 25, 25, 3, 3, (1, 1), (2, 2, 1, 1), (2, 1), False, False),    # dilated rows only: halo form
    (2, 32, 17, 40, 3, 3, (1, 2), (1, 1, 1, 1), (1, 1), True, False),     # stride along the width only
    (1, 32, 9, 70000 // 9, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), True, False),   # a very wide map
]


@pytest.mark.parametrize("case", DEPTHWISE_ROWS)
def test_conv_depthwise_row_segments(ctx, case):
    n, c, ih, iw, kh, kw, stride, pads, dil, relu, with_table = case
    rng = np.random.default_rng(c + kh * 7 + kw + iw)
    x = rnd_i8(rng, (n, c, ih, iw))
    w = rnd_w(rng, (c, 1, kh, kw), 24)
    bias, rsh, mult = rnd_params(rng, c, 5, 12, 2048)
    want = oracle_conv(x, w, bias, rsh, mult, c, stride, pads, dil, (0, 0), relu)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=capi.ALGO_DEPTHWISE, g=c, stride=stride, pads=pads,
                         dil=dil, do_relu=relu)
    assert name == "depthwise" and np.array_equal(got, want)
    assert len(np.unique(want)) > 8
    if with_table:
        table = rnd_i8(rng, 256)
        table[0] = 9
        d = conv_desc(x.shape, w.shape, g=c, stride=stride, pads=pads, dil=dil, do_relu=relu, algo=capi.ALGO_DEPTHWISE)
        wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
        xt, yt, tt = ctx.from_nchw(x), ctx.tensor(want.shape), ctx.tensor(want.shape)
        ctx.conv_post(wh, xt, yt, table, tt)
        assert np.array_equal(ctx.to_nchw(yt), want)
        assert np.array_equal(ctx.to_nchw(tt), O.lut_i8(want, table))
        assert tt.cs == c or not ctx.raw(tt)[..., c:].any()
        # the table's result alone: the conv result is not written
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, tt.ptr, 0x33, tt.nbytes))
        ctx.conv_post(wh, xt, None, table, tt)
        assert (ctx.raw(yt) == 0x55).all()
        assert np.array_equal(ctx.to_nchw(tt), O.lut_i8(want, table))
        ctx.conv_weights_destroy(wh)
        for t in (xt, yt, tt):
            t.free()


@pytest.mark.parametrize("algo", [capi.ALGO_DEPTHWISE, capi.ALGO_DEPTHWISE_DOT])
def test_conv_depthwise_dilated_general_requant_and_fused_table(ctx, algo):
    rng = np.random.default_rng(77)
    x = rnd_i8(rng, (2, 40, 14, 13))
    w = rnd_w(rng, (40, 1, 3, 3), 24)
    bias, rsh, mult = rnd_params(rng, 40, 5, 12, 2048)
    rsh[3] = 0                                         # forces the general rounding form
    want = oracle_conv(x, w, bias, rsh, mult, 40, (1, 1), (2, 2, 2, 2), (2, 2), (0, 0), True)
    got, name = run_conv(ctx, x, w, bias, rsh, mult, algo=algo, g=40, pads=(2, 2, 2, 2), dil=(2, 2),
                         do_relu=True)
    assert name.startswith("depthwise") and np.array_equal(got, want)
    # the same layer with a table behind it, in one kernel
    table = rnd_i8(rng, 256)
    table[0] = -5
    d = conv_desc(x.shape, w.shape, g=40, pads=(2, 2, 2, 2), dil=(2, 2), do_relu=True, algo=algo)
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    xt, yt, tt = ctx.from_nchw(x), ctx.tensor(want.shape), ctx.tensor(want.shape)
    ctx.conv_post(wh, xt, yt, table, tt)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert np.array_equal(ctx.to_nchw(tt), O.lut_i8(want, table))
    assert not ctx.raw(tt)[..., 40:].any()
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    ctx.conv_post(wh, xt, None, table, tt)
    assert (ctx.raw(yt) == 0x55).all()
    ctx.conv_weights_destroy(wh)


def test_conv_grouped_and_inserted_zeros_direct(ctx):
    rng = np.random.default_rng(3)
    x = rnd_i8(rng, (2, 12, 7, 6))
    w = rnd_w(rng, (8, 3, 3, 3))
    bias, rsh, mult = rnd_params(rng, 8, 4, 9)
    want = oracle_conv(x, w, bias, rsh, mult, 4, (1, 1), (1, 1, 1, 1))
    got, _ = run_conv(ctx, x, w, bias, rsh, mult, g=4, pads=(1, 1, 1, 1))
    assert np.array_equal(got, want)
    w2 = rnd_w(rng, (5, 12, 3, 3))
    bias, rsh, mult = rnd_params(rng, 5, 6, 10)
    want = oracle_conv(x, w2, bias, rsh, mult, 1, (1, 1), (1, 1, 1, 1), (1, 1), (1, 2))
    got, name = run_conv(ctx, x, w2, bias, rsh, mult, pads=(1, 1, 1, 1), ins=(1, 2))
    assert name == "direct" and np.array_equal(got, want)


def test_conv_without_bias_and_null_bias(ctx):
    rng = np.random.default_rng(5)
    x = rnd_i8(rng, (1, 16, 6, 6))
    w = rnd_w(rng, (16, 16, 3, 3))
    bias, rsh, mult = rnd_params(rng, 16)
    want = oracle_conv(x, w, bias, rsh, mult, pads=(1, 1, 1, 1), with_bias=False)
    got, _ = run_conv(ctx, x, w, bias, rsh, mult, pads=(1, 1, 1, 1), with_bias=False)
    assert np.array_equal(got, want)
    got, _ = run_conv(ctx, x, w, None, rsh, mult, pads=(1, 1, 1, 1), with_bias=True)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("algo", [capi.ALGO_MFMA, capi.ALGO_DIRECT])
def test_conv_requant_edge_parameters(ctx, algo):
    """rshift 0 and 31, multipliers that are not float32-exact, zero, 2^31 (which the
    reference turns into INT_MIN) and large accumulators."""
    rng = np.random.default_rng(7)
    oc = 32
    x = rnd_i8(rng, (1, 256, 4, 4), 100, 127)
    w = rnd_i8(rng, (oc, 256, 3, 3), 100, 127)       # sums near 9*256*127*127 = 3.7e7
    w[1::2] = -w[1::2]
    bias = rng.integers(-(1 << 23), 1 << 23, oc).astype(np.float32)
    mult = (rng.integers(1 << 30, (1 << 31) - 1, oc)).astype(np.float32)   # rounded by float32
    mult[0] = 0
    mult[1] = float(2 ** 31)       # -> uint32 2^31 -> int32 INT_MIN
    mult[2] = 1.0
    mult[3] = float((1 << 31) - 1)  # rounds up to 2^31 as a float
    rsh = rng.integers(0, 32, oc).astype(np.float32)
    rsh[4], rsh[5], rsh[6], rsh[7] = 0, 31, 1, 30
    want = oracle_conv(x, w, bias, rsh, mult, pads=(1, 1, 1, 1))
    got, _ = run_conv(ctx, x, w, bias, rsh, mult, algo=algo, pads=(1, 1, 1, 1))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("tile", [0, 2, 7, 9, 13, 16])   # persistent, wide K, one-tile, LDS-free, split K
@pytest.mark.parametrize("relu,rs,keep_y", [(True, 6, True), (False, 0, True), (True, 9, False)])
def test_conv_with_fused_eltwise_add(ctx, tile, relu, rs, keep_y):
    """conv + EltwiseAdd in one kernel == the two ops run one after the other"""
    rng = np.random.default_rng(tile * 31 + rs)
    x = rnd_i8(rng, (2, 64, 13, 11))
    w = rnd_w(rng, (72, 64, 3, 3))
    bias, rsh, mult = rnd_params(rng, 72)
    other = rnd_i8(rng, (2, 72, 13, 11))
    m_src, m_conv = int(rng.integers(-100, 100)), int(rng.integers(20, 100))
    y_ref = oracle_conv(x, w, bias, rsh, mult, 1, (1, 1), (1, 1, 1, 1))
    z_ref = O.eltwise_add_i8([other, y_ref], [m_src, m_conv], [rs], relu)
    d = conv_desc(x.shape, w.shape, pads=(1, 1, 1, 1), algo=16 + tile)
    xt, ot = ctx.from_nchw(x), ctx.from_nchw(other)
    yt, zt = ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    ctx.conv_add(wh, xt, yt if keep_y else None, ot, zt, m_src, m_conv, rs, relu)
    assert np.array_equal(ctx.to_nchw(zt), z_ref)
    assert not ctx.raw(zt)[..., 72:].any()
    if keep_y:
        assert np.array_equal(ctx.to_nchw(yt), y_ref)
    else:
        assert (ctx.raw(yt) == 0x55).all()      # the conv result was not written
    ctx.conv_weights_destroy(wh)


@pytest.mark.parametrize("tile", [0, 1, 3, 6, 9, 12])      # the variants with an LDS epilogue
@pytest.mark.parametrize("with_add,keep_y,keep_lut", [(False, True, True), (False, False, True),
                                                      (True, True, True), (True, False, False)])
def test_conv_with_fused_table_and_add(ctx, tile, with_add, keep_y, keep_lut):
    """conv -> 256-entry table -> EltwiseAdd in one kernel == the three ops one after the other"""
    rng = np.random.default_rng(tile * 17 + with_add * 5 + keep_y)
    x = rnd_i8(rng, (2, 48, 13, 11))
    w = rnd_w(rng, (72, 48, 3, 3))                # 72 channels: 8 pad channels in the last group
    bias, rsh, mult = rnd_params(rng, 72)
    table = rnd_i8(rng, 256)
    table[0] = 77                                  # pad channels must stay 0 all the same
    other = rnd_i8(rng, (2, 72, 13, 11))
    y_ref = oracle_conv(x, w, bias, rsh, mult, 1, (1, 1), (1, 1, 1, 1))
    t_ref = O.lut_i8(y_ref, table)
    z_ref = O.eltwise_add_i8([other, t_ref], [37, 51], [6], True)
    d = conv_desc(x.shape, w.shape, pads=(1, 1, 1, 1), algo=16 + tile)
    xt, ot = ctx.from_nchw(x), ctx.from_nchw(other)
    yt, tt, zt = ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape), ctx.tensor(y_ref.shape)
    for t in (yt, tt, zt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    wh = ctx.conv_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    ctx.conv_post(wh, xt, yt if keep_y else None, table, tt if keep_lut else None,
                  (ot, zt, 37, 51, 6, True) if with_add else None)
    if keep_y:
        assert np.array_equal(ctx.to_nchw(yt), y_ref)
    else:
        assert (ctx.raw(yt) == 0x55).all()
    if keep_lut:
        assert np.array_equal(ctx.to_nchw(tt), t_ref)
        assert not ctx.raw(tt)[..., 72:].any()
    else:
        assert (ctx.raw(tt) == 0x55).all()
    if with_add:
        assert np.array_equal(ctx.to_nchw(zt), z_ref)
        assert not ctx.raw(zt)[..., 72:].any()
    ctx.conv_weights_destroy(wh)


def test_conv_table_fusion_needs_an_lds_variant(ctx):
    d = conv_desc((1, 32, 6, 6), (32, 32, 1, 1), algo=16 + 13)      # LDS-free variant
    wh = ctx.conv_prepack(d, np.ones((32, 32, 1, 1), np.int8), None, np.full(32, 1 << 30, np.int32),
                          np.full(32, 8, np.int32))
    xt, yt = ctx.tensor((1, 32, 6, 6)), ctx.tensor((1, 32, 6, 6))
    with pytest.raises(capi.TpuHipError, match="cannot fuse a table"):
        ctx.conv_post(wh, xt, yt, np.zeros(256, np.int8), yt)
    with pytest.raises(capi.TpuHipError, match="nothing would be written"):
        ctx.conv_post(wh, xt, None)
    ctx.conv_weights_destroy(wh)


def test_conv_rejects_bad_arguments(ctx):
    d = conv_desc((1, 16, 4, 4), (16, 16, 3, 3), pads=(1, 1, 1, 1))
    w = np.zeros((16, 16, 3, 3), np.int8)
    ok = np.zeros(16, np.int32)
    bad = ok.copy()
    bad[3] = 32
    with pytest.raises(capi.TpuHipError, match="rshift"):
        ctx.conv_prepack(d, w, None, ok, bad)
    d2 = conv_desc((1, 16, 4, 4), (16, 16, 3, 3), pads=(1, 1, 1, 1), out_hw=(9, 9))
    with pytest.raises(capi.TpuHipError, match="window"):
        ctx.conv_prepack(d2, w, None, ok, ok)
    d3 = conv_desc((1, 16, 4, 4), (16, 4, 3, 3), g=4, pads=(1, 1, 1, 1), algo=capi.ALGO_MFMA)
    with pytest.raises(capi.TpuHipError, match="MFMA"):
        ctx.conv_prepack(d3, np.zeros((16, 4, 3, 3), np.int8), None, ok, ok)


@pytest.mark.parametrize("m,k,n,relu", [(32, 2048, 1000, False), (5, 100, 37, True),
                                        (64, 1280, 1000, True),
                                        # the one-launch kernel (K of 1024 and more): exactly one K step
                                        # per wave, waves left without work, an odd number of steps per
                                        # wave, ragged rows and channels
                                        (1, 1024, 10, False), (33, 1090, 65, True), (7, 3100, 40, False),
                                        (256, 1500, 96, True), (40, 4160, 33, False),
                                        # the two-launch kernels just below that K
                                        (17, 1000, 70, True),
                                        # more input channels than the conv kernels index (the first
                                        # classifier layers of VGG / AlexNet): few rows, and more rows
                                        # than the K-splitting kernels otherwise take
                                        (4, 9216, 50, True), (2, 25088, 64, False), (300, 4112, 40, True)])
def test_fully_connected(ctx, m, k, n, relu):
    rng = np.random.default_rng(m + k + n)
    x = rnd_i8(rng, (m, k))
    w = rnd_w(rng, (n, k), 20 if k <= 4160 else 4)     # sums the reference's fp32 holds exactly
    bias = rng.integers(-3000, 3000, n).astype(np.float32)
    mult, rsh = np.float32((1 << 30) + 128 * 12345), np.float32(9 if k <= 4160 else 10)
    want = O.fc_i8(x, w, bias, [rsh], [mult], 1, m, k, n, relu)[0]
    xt = ctx.from_nchw(x.reshape(m, k, 1, 1))
    yt = ctx.tensor((m, n, 1, 1))
    wh = ctx.fc_prepack(m, k, n, xt.cs, yt.cs, relu, w, f2i32(bias), f2i32([mult])[0],
                        f2i32([rsh])[0])
    ctx.conv(wh, xt, yt)
    got = ctx.to_nchw(yt).reshape(m, n)
    assert np.array_equal(got, want)
    # the FullyConnected entry point: the K-splitting kernels for matrices of few rows
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    ctx.fc(wh, xt, yt)
    assert np.array_equal(ctx.to_nchw(yt).reshape(m, n), want)
    assert O.fc_guard(x, w, bias, 1, m, k, n) < (1 << 24)
    ctx.conv_weights_destroy(wh)


def _view4(shape):
    return tuple(shape) + (1,) * (4 - len(shape))


@pytest.mark.parametrize("bh,bl,m,k,n,lt,ot,relu", [
    (1, 4, 3, 28, 5, 0, 0, False),     # [4,3,28] x [4,5,28] -> [4,3,5] (TPUOperationSupport.cpp:566)
    (1, 6, 17, 64, 33, 0, 0, True),
    (2, 3, 8, 48, 20, 1, 0, True),     # input [2,8,3,48]
    (2, 3, 8, 48, 20, 0, 1, False),    # result [2,8,3,20]
    (3, 2, 5, 40, 7, 1, 1, True),
    (1, 1, 12, 28, 5, 0, 0, False),    # [4,3,28] x [5,28] -> [4,3,5]: one matmul, rank-3 result
])
def test_fully_connected_batched_and_transposed(ctx, bh, bl, m, k, n, lt, ot, relu):
    """core/fullyconnected.cpp:52-88 through tpuhip_fc_batched_i8: tensors lie channels-last on the
    device in the 4-d views of their logical shapes, the kernel finds its operands through them"""
    rng = np.random.default_rng(bh * 1000 + bl * 100 + m + k + n + lt * 7 + ot * 13)
    batch = bh * bl
    if bh == bl == 1:
        x_shape, y_shape = (4, m // 4, k), (4, m // 4, n)
    else:
        x_shape = (bh, m, bl, k) if lt else ((bh, bl, m, k) if bh > 1 else (batch, m, k))
        y_shape = (bh, m, bl, n) if ot else ((bh, bl, m, n) if bh > 1 else (batch, m, n))
    x = rnd_i8(rng, x_shape)
    w = rnd_w(rng, (batch, n, k), 20)
    bias = rng.integers(-3000, 3000, (batch, n)).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, batch) * 128).astype(np.float32)
    rsh = rng.integers(6, 11, batch).astype(np.float32)
    want = O.fc_batched_i8(x, w, bias, rsh, mult, bh, bl, m, k, n, lt, ot, relu).reshape(y_shape)
    xt = ctx.from_nchw(x.reshape(_view4(x_shape)))
    yt = ctx.tensor(_view4(y_shape))
    xv, yv = _view4(x_shape), _view4(y_shape)
    d = capi.FcBatchedDesc(bh, bl, m, k, n, lt, ot, int(relu), xv[1], xv[2], xv[3], xt.cs,
                           yv[1], yv[2], yv[3], yt.cs)
    wh = ctx.fc_batched_prepack(d, w, f2i32(bias), f2i32(mult), f2i32(rsh))
    ctx.fc_batched(wh, xt, yt)
    got = ctx.to_nchw(yt).reshape(y_shape)
    assert np.array_equal(got, want)
    assert len(np.unique(want)) > 8
    ctx.fc_batched_destroy(wh)


def test_fully_connected_batched_refuses_bad_descriptors(ctx):
    ok = np.zeros(2, np.int32)
    w = np.zeros((2, 4, 8), np.int8)
    good = dict(batch_high=1, batch_low=2, m=3, k=8, n=4, input_transpose=0, output_transpose=0, do_relu=0,
                x_c=3, x_h=8, x_w=1, x_cs=16, y_c=3, y_h=4, y_w=1, y_cs=16)
    for bad, msg in ((dict(k=0), "positive"), (dict(x_h=7), "divide"), (dict(x_h=4, x_w=2), "last dim"),
                     (dict(y_h=2, y_w=2), "last dim"), (dict(x_cs=2), "channel stride")):
        with pytest.raises(capi.TpuHipError, match=msg):
            ctx.fc_batched_prepack(capi.FcBatchedDesc(**dict(good, **bad)), w, None, ok, ok)
    with pytest.raises(capi.TpuHipError, match="rshift"):
        ctx.fc_batched_prepack(capi.FcBatchedDesc(**good), w, None, ok, np.array([3, 40], np.int32))


@pytest.mark.parametrize("nin,relu,rs", [(2, True, 5), (2, False, 0), (3, False, 7), (1, True, 2),
                                         (8, True, 9)])
def test_eltwise_add(ctx, nin, relu, rs):
    rng = np.random.default_rng(nin * 10 + rs)
    shape = (2, 24, 7, 9)
    xs = [rnd_i8(rng, shape) for _ in range(nin)]
    mult = rng.integers(-128, 128, nin).astype(np.float32)
    want = O.eltwise_add_i8(xs, mult, [rs], relu)
    ts = [ctx.from_nchw(a) for a in xs]
    yt = ctx.tensor(shape)
    ctx.eltwise_add(ts, mult.astype(np.int8), rs, relu, yt)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., 24:].any()


@pytest.mark.parametrize("k,s,pads,shape,out_hw", [
    ((3, 3), (2, 2), (0, 1, 0, 1), (2, 64, 28, 28), None),   # ResNet-50 pool1 (Caffe ceil mode)
    ((3, 3), (2, 2), (1, 1, 1, 1), (1, 24, 9, 11), None),
    ((2, 2), (2, 2), (0, 0, 0, 0), (1, 5, 8, 8), None),
    ((3, 2), (1, 2), (1, 0, 0, 1), (1, 40, 7, 9), None),
])
def test_pool_max(ctx, k, s, pads, shape, out_hw):
    rng = np.random.default_rng(sum(shape))
    x = rnd_i8(rng, shape)
    want = O.pool_max_i8(x, O.make_pool_desc(shape, k, s, pads, out_hw))
    d = pool_desc(shape, k, s, pads, out_hw)
    xt = ctx.from_nchw(x)
    yt = ctx.tensor((d.n, d.c, d.oh, d.ow))
    ctx.pool_max(d, xt, yt)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., shape[1]:].any()


@pytest.mark.parametrize("k,s,pads,shape,mult,rs", [
    ((7, 7), (1, 1), (0, 0, 0, 0), (4, 2048, 7, 7), 167, 13),   # ResNet-50 global average
    ((7, 7), (1, 1), (0, 0, 0, 0), (2, 1280, 7, 7), 84, 12),
    ((3, 3), (2, 2), (1, 1, 1, 1), (1, 20, 9, 9), 57, 9),
    ((2, 2), (2, 2), (0, 0, 0, 0), (1, 3, 6, 6), 1, 0),
    ((3, 3), (1, 1), (1, 1, 1, 1), (1, 16, 5, 5), 255, 3),      # saturates
])
def test_pool_avg(ctx, k, s, pads, shape, mult, rs):
    rng = np.random.default_rng(sum(shape) + mult)
    x = rnd_i8(rng, shape)
    want = O.pool_avg_i8(x, O.make_pool_desc(shape, k, s, pads), rs, mult)
    d = pool_desc(shape, k, s, pads)
    xt = ctx.from_nchw(x)
    yt = ctx.tensor((d.n, d.c, d.oh, d.ow))
    ctx.pool_avg(d, xt, yt, mult, rs)
    assert np.array_equal(ctx.to_nchw(yt), want)


def test_leaky_relu_lut_relu(ctx):
    rng = np.random.default_rng(41)
    shape = (2, 40, 6, 5)
    x = rnd_i8(rng, shape)
    x.reshape(-1)[:256] = np.arange(-128, 128)      # every input value occurs
    xt = ctx.from_nchw(x)
    yt = ctx.tensor(shape)
    for rp, mp, rn, mn in ((0, 1, 7, 13), (5, 33, 10, 102), (0, 0, 6, 6)):
        ctx.leaky_relu(xt, yt, rp, mp, rn, mn)
        assert np.array_equal(ctx.to_nchw(yt), O.leaky_relu_i8(x, rp, mp, rn, mn))
        assert not ctx.raw(yt)[..., 40:].any()
    table = rng.integers(-128, 128, 256).astype(np.int8)
    ctx.lut(xt, yt, table)
    assert np.array_equal(ctx.to_nchw(yt), O.lut_i8(x, table.astype(np.float32)))
    assert not ctx.raw(yt)[..., 40:].any()       # table[0] != 0 must not leak into the pads
    ctx.relu(xt, yt)
    assert np.array_equal(ctx.to_nchw(yt), O.relu_i8(x))
    ctx.lut(xt, yt, ctx.clip_table(0, 77, 0, 1))
    assert np.array_equal(ctx.to_nchw(yt), O.clip_i8(x, 0, 77, 0, 1))


def test_upsample(ctx):
    rng = np.random.default_rng(43)
    for shape, sh, sw in (((2, 256, 19, 19), 2, 2), ((1, 24, 5, 4), 3, 1), ((1, 8, 3, 3), 1, 2)):
        x = rnd_i8(rng, shape)
        xt = ctx.from_nchw(x)
        yt = ctx.tensor((shape[0], shape[1], shape[2] * sh, shape[3] * sw))
        ctx.upsample(xt, yt, sh, sw)
        assert np.array_equal(ctx.to_nchw(yt), O.upsample_i8(x, sh, sw))


@pytest.mark.parametrize("axis", [0, 1, 2, 3])
def test_concat_axes(ctx, axis):
    rng = np.random.default_rng(47 + axis)
    base = [2, 32, 5, 6]
    shapes = []
    # three inputs that change no byte: one launch along any axis
    for extent in (3, 1, 4) if axis != 1 else (32, 16, 48):
        s = list(base)
        s[axis] = extent
        shapes.append(tuple(s))
    xs = [rnd_i8(rng, s) for s in shapes]
    want = O.concat_i8(xs, axis)
    ts = [ctx.from_nchw(a) for a in xs]
    yt = ctx.tensor(want.shape)
    ctx.concat(ts, axis, yt)
    assert np.array_equal(ctx.to_nchw(yt), want)


@pytest.mark.parametrize("channels, in_cs, y_cs", [((16, 48), (None, None), None), ((32, 16, 16, 64), (None, 32, None, 80), None),
                                                   ((128, 256), (None, None), 400), ((16, 16, 16, 16, 16), (None,) * 5, None)])
def test_concat_whole_channel_groups(ctx, channels, in_cs, y_cs):
    """channel concat of inputs with whole 16-channel groups (one launch for two to four inputs; the fifth
    case has too many and takes a launch per input), with padded strides on either side and identity rescaling"""
    rng = np.random.default_rng(131 + len(channels))
    xs = [rnd_i8(rng, (2, c, 7, 9)) for c in channels]
    want = O.concat_i8(xs, 1)
    ts = [ctx.from_nchw(a, cs) for a, cs in zip(xs, in_cs)]
    yt = ctx.tensor(want.shape, y_cs)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))   # poison: the pad channels must be written
    ctx.concat(ts, 1, yt, [0] * len(xs), [1] * len(xs), False)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., want.shape[1]:].any()
    for t in ts + [yt]:
        t.free()


def test_concat_channels_unaligned_requant_relu(ctx):
    rng = np.random.default_rng(53)
    xs = [rnd_i8(rng, (2, c, 4, 5)) for c in (24, 7, 40)]
    rsh, mult = [0, 3, 6], [1, 5, 77]
    want = O.concat_i8(xs, 1, rsh, mult, True)
    ts = [ctx.from_nchw(a) for a in xs]
    yt = ctx.tensor(want.shape)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    ctx.concat(ts, 1, yt, rsh, mult, True)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., 71:].any()


def test_layout_round_trip_and_float_edge(ctx):
    rng = np.random.default_rng(59)
    x = rnd_i8(rng, (3, 37, 11, 13))
    t = ctx.from_nchw(x)
    raw = ctx.raw(t)
    assert np.array_equal(raw[..., :37], x.transpose(0, 2, 3, 1))
    assert not raw[..., 37:].any()
    assert np.array_equal(ctx.to_nchw(t), x)
    # float-stored edge
    xf = x.astype(np.float32)
    src = ctx.malloc(xf.nbytes)
    ctx.upload(src, xf)
    t2 = ctx.tensor(x.shape)
    n, c, h, w = x.shape
    ctx._ck(ctx.lib.tpuhip_nchw_f32_to_nhwc_i8(ctx.h, src, t2.ptr, n, c, h, w, t2.cs))
    assert np.array_equal(ctx.raw(t2), raw)
    dst = ctx.malloc(xf.nbytes)
    ctx._ck(ctx.lib.tpuhip_nhwc_i8_to_nchw_f32(ctx.h, t2.ptr, dst, n, c, h, w, t2.cs))
    assert np.array_equal(ctx.download(dst, x.shape, np.float32), xf)


BINARY_SHAPES = [((2, 40, 9, 7), (2, 40, 9, 7)),      # same shape (the Eltwise* ops)
                 ((2, 40, 9, 7), (1, 40, 1, 1)),      # per-channel operand (scale-like)
                 ((2, 40, 9, 7), (2, 1, 9, 7)),       # one channel repeated over all
                 ((1, 1, 9, 1), (2, 40, 1, 7)),       # both operands broadcast
                 ((2, 40, 1, 1), (2, 40, 9, 7)),      # squeeze-excite gate times feature map
                 ((3, 16, 4, 4), (1, 1, 1, 1))]       # scalar


@pytest.mark.parametrize("shapes", BINARY_SHAPES)
@pytest.mark.parametrize("op", [capi.BIN_ADD, capi.BIN_SUB, capi.BIN_MAX, capi.BIN_MIN, capi.BIN_MUL])
@pytest.mark.parametrize("relu", [False, True])
def test_binary_ops_with_broadcast(ctx, shapes, op, relu):
    rng = np.random.default_rng(op * 13 + len(shapes[0]) + relu)
    a, b = rnd_i8(rng, shapes[0]), rnd_i8(rng, shapes[1])
    out_shape = tuple(max(p, q) for p, q in zip(*shapes))
    at, bt, yt = ctx.from_nchw(a), ctx.from_nchw(b), ctx.tensor(out_shape)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    if op == capi.BIN_MUL:
        for mult, r in [(1 << 30, 7), (1518500250, 6), ((1 << 31) - 128, 14), (1 << 30, 0)]:
            want = O.binary_i8(op, a, b, [float(mult)], r, relu)
            ctx.binary(op, at, bt, yt, multiplier=f2i32(np.float32(mult)), rshift=r, do_relu=relu)
            assert np.array_equal(ctx.to_nchw(yt), want), (mult, r)
    else:
        for m0, m1, r in [(1, 1, 0), (3, -2, 1), (127, 127, 7), (-128, 77, 8), (90, 45, 30)]:
            want = O.binary_i8(op, a, b, [m0, m1], r, relu)
            ctx.binary(op, at, bt, yt, m0=m0, m1=m1, rshift=r, do_relu=relu)
            assert np.array_equal(ctx.to_nchw(yt), want), (m0, m1, r)
    assert not ctx.raw(yt)[..., out_shape[1]:].any()        # pad channels written as zero


def test_binary_rejects_bad_arguments(ctx):
    a, b = ctx.tensor((1, 16, 4, 4)), ctx.tensor((1, 8, 4, 4))
    with pytest.raises(capi.TpuHipError, match="neither 1 nor"):
        ctx.binary(capi.BIN_ADD, a, b, a)
    with pytest.raises(capi.TpuHipError, match="no int8 meaning"):
        ctx.binary(capi.BIN_MUL, a, a, a, multiplier=0, rshift=0)
    with pytest.raises(capi.TpuHipError, match="int8"):
        ctx.binary(capi.BIN_MAX, a, a, a, m0=300)


@pytest.mark.parametrize("shape", [(2, 7, 256, 1), (3, 40, 9, 11), (1, 130, 5, 5)])
def test_prelu_per_channel_tables(ctx, shape):
    rng = np.random.default_rng(shape[1])
    x = rnd_i8(rng, shape)
    if shape[2] == 256:
        x[...] = np.arange(-128, 128, dtype=np.int8).reshape(1, 1, 256, 1)    # every input value
    slope = rng.integers(-128, 128, shape[1]).astype(np.float32)
    xt, yt = ctx.from_nchw(x), ctx.tensor(shape)
    for mp, rp, rn in [(1, 0, 0), (3, 1, 2), (200, 7, 5)]:
        ctx.prelu(xt, yt, slope, rp, mp, rn)
        assert np.array_equal(ctx.to_nchw(yt), O.prelu_i8(x, slope, rp, mp, rn)), (mp, rp, rn)
        assert not ctx.raw(yt)[..., shape[1]:].any()


MOVES = [
    ("pad_const", (2, 20, 5, 4), [0, 1, 2, 3, 1, 0, 4, 1], None),
    ("pad_const", (2, 20, 5, 4), [0, -1, 2, -2, 0, 1, -1, 0], None),
    ("pad_edge", (2, 20, 5, 4), [0, 0, 2, 1, 0, 0, 3, 4], None),
    ("crop", (3, 37, 9, 8), [1, 2, 0, 3, 1, 1, 1, 1], (2, 30, 9, 5)),
    ("crop", (3, 37, 9, 8), [0, 1, 2, 0, 2, 3, 2, 4], (2, 12, 4, 2)),
    ("permute", (2, 3, 18, 4), [0, 2, 3, 1], None),
    ("permute", (2, 19, 5, 4), [0, 3, 1, 2], None),
    ("permute", (4, 3, 5, 33), [3, 2, 1, 0], None),
    ("reorg", (2, 24, 6, 4), [2], None),
    ("tile", (2, 20, 5, 4), [1, 3], None),
    ("tile", (2, 20, 5, 4), [3, 2], None),
    ("reverse", (2, 20, 5, 4), [1], None),
    ("reverse", (2, 20, 5, 4), [2], None),
    ("shuffle_channel", (2, 24, 3, 4), [3], None),
    ("depth_to_space", (2, 36, 3, 4), [3, 0], None),
    ("depth_to_space", (2, 64, 3, 4), [2, 1], None),
    ("dilate", (2, 20, 5, 4), [1, 2, -7], None),       # ins_w, ins_h, fill_constant
    ("dilate", (1, 3, 6, 7), [3, 0, 0], None),
    ("dilate", (2, 17, 1, 9), [0, 0, 5], None),        # nothing inserted: a copy
    ("reflection_pad", (2, 20, 5, 6), [2, 5], None),
    ("reflection_pad", (1, 3, 4, 9), [0, 8], None),
    ("reflection_pad", (3, 33, 2, 2), [1, 1], None),
]


@pytest.mark.parametrize("kind,shape,params,out_shape", MOVES)
def test_data_movement_ops(ctx, kind, shape, params, out_shape):
    rng = np.random.default_rng(len(kind) + shape[1])
    x = rnd_i8(rng, shape)
    want = O.move_i8(kind, x, params, out_shape)
    xt, yt = ctx.from_nchw(x), ctx.tensor(want.shape)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    ctx.move(O.MOVE_KINDS.index(kind), xt, yt, params)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., want.shape[1]:].any()


@pytest.mark.parametrize("x_cs,y_cs", [(32, 48), (48, 32), (32, 32), (64, 32)])
def test_permute_that_keeps_the_channels_with_padded_strides(ctx, x_cs, y_cs):
    """order (0, 1, 3, 2): a pixel's channel row moves as 16-byte groups; with a wider stride on either
    side no group may come from the neighbouring pixel, and the output's pad groups must be zero"""
    rng = np.random.default_rng(x_cs * 3 + y_cs)
    shape = (2, 20, 5, 7)
    x = rnd_i8(rng, shape)
    want = O.move_i8("permute", x, [0, 1, 3, 2], None)
    xt, yt = ctx.from_nchw(x, cs=x_cs), ctx.tensor(want.shape, cs=y_cs)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    ctx.move(O.MOVE_KINDS.index("permute"), xt, yt, [0, 1, 3, 2])
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., shape[1]:].any()


def test_data_movement_rejects_bad_arguments(ctx):
    x, y = ctx.tensor((1, 16, 4, 4)), ctx.tensor((1, 16, 4, 4))
    with pytest.raises(capi.TpuHipError, match="reads past"):
        ctx.move(capi.MOVE_CROP, x, y, [0, 1, 0, 0, 1, 1, 1, 1])
    with pytest.raises(capi.TpuHipError, match="permutation"):
        ctx.move(capi.MOVE_PERMUTE, x, y, [0, 1, 2, 2])
    with pytest.raises(capi.TpuHipError, match="no int8 value"):
        ctx.move(O.MOVE_KINDS.index("dilate"), x, ctx.tensor((1, 16, 7, 7)), [1, 1, 200])
    with pytest.raises(capi.TpuHipError, match="dilate: output shape"):
        ctx.move(O.MOVE_KINDS.index("dilate"), x, ctx.tensor((1, 16, 8, 8)), [1, 1, 0])
    with pytest.raises(capi.TpuHipError, match="reflection_pad: pads"):
        ctx.move(O.MOVE_KINDS.index("reflection_pad"), x, ctx.tensor((1, 16, 4, 9)), [4, 1])
    with pytest.raises(capi.TpuHipError, match="group"):
        ctx.move(capi.MOVE_SHUFFLE_CHANNEL, x, y, [5])
    with pytest.raises(capi.TpuHipError, match="expected"):
        ctx.move(capi.MOVE_PAD_CONST, x, y, [0, 0, 1, 0, 0, 0, 0, 0])


@pytest.mark.parametrize("shape,local_size,sum_rshift,lrn_rshift,q0,q1", [
    ((2, 64, 9, 7), 5, 8, 9, 120, 93),
    ((1, 21, 5, 5), 3, 0, 3, 1, 2),          # channels not a multiple of 4 or 16
    ((3, 192, 4, 6), 5, 11, 12, 200, 255),
    ((1, 4, 3, 3), 7, 6, 9, 64, 2),          # window wider than the tensor
])
def test_lrn_matches_the_oracle(ctx, shape, local_size, sum_rshift, lrn_rshift, q0, q1):
    rng = np.random.default_rng(shape[1] + local_size)
    x = rnd_i8(rng, shape)
    sq, pw = rng.integers(0, 256, 256), rng.integers(0, 256, 256)
    want = O.lrn_i8(x, local_size, sq, pw, sum_rshift, lrn_rshift, q0, q1)
    xt, yt = ctx.from_nchw(x), ctx.tensor(shape)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))
    ctx.lrn(xt, yt, local_size, sq, pw, sum_rshift, lrn_rshift, q0, q1)
    assert np.array_equal(ctx.to_nchw(yt), want)
    assert not ctx.raw(yt)[..., shape[1]:].any()          # pad channels rewritten as zero
    assert len(np.unique(want)) > 8


def test_lrn_refuses_parameters_whose_float_form_is_inexact(ctx):
    xt, yt = ctx.tensor((1, 16, 2, 2)), ctx.tensor((1, 16, 2, 2))
    t = np.zeros(256, np.uint8)
    with pytest.raises(capi.TpuHipError, match="quant_data0"):
        ctx.lrn(xt, yt, 5, t, t, 8, 8, 20000, 10)
    with pytest.raises(capi.TpuHipError, match="quant_data1"):
        ctx.lrn(xt, yt, 5, t, t, 8, 8, 100, 600)
    with pytest.raises(capi.TpuHipError, match="local_size"):
        ctx.lrn(xt, yt, 0, t, t, 8, 8, 100, 100)


def test_random_pool_add_table_upsample_concat_sweep(ctx):
    """700 random cases over max / average pooling (windows, strides, pads, global), n-input add,
    byte tables, leaky relu, upsample and concat (with and without rescaling) against the oracle"""
    seen = {}
    for it in range(700):
        rng = np.random.default_rng(888000 + it)
        kind = ["max", "avg", "add", "lut", "leaky", "up", "concat"][int(rng.integers(0, 7))]
        n, c, ih, iw = int(rng.integers(1, 4)), int(rng.integers(1, 150)), int(rng.integers(1, 30)), int(rng.integers(1, 30))
        x = rnd_i8(rng, (n, c, ih, iw))
        xt = ctx.from_nchw(x)
        tmp = [xt]
        try:
            if kind in ("max", "avg"):
                if rng.integers(0, 5) == 0:
                    k, s, pads = (ih, iw), (1, 1), (0, 0, 0, 0)
                else:
                    k = (int(rng.integers(1, 5)), int(rng.integers(1, 5)))
                    s = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
                    pads = tuple(int(min(v, kk - 1)) for v, kk in zip(rng.integers(0, 3, 4), (k[0], k[0], k[1], k[1])))
                if ih + pads[0] + pads[1] < k[0] or iw + pads[2] + pads[3] < k[1]:
                    continue
                d0, d = O.make_pool_desc(x.shape, k, s, pads), pool_desc(x.shape, k, s, pads)
                yt = ctx.tensor((n, c, d0.oh, d0.ow))
                tmp.append(yt)
                if kind == "max":
                    want = O.pool_max_i8(x, d0)
                    ctx.pool_max(d, xt, yt)
                else:
                    mult, rs = int(rng.integers(1, 256)), int(rng.integers(0, 14))
                    want = O.pool_avg_i8(x, d0, rs, mult)
                    ctx.pool_avg(d, xt, yt, mult, rs)
            elif kind == "add":
                nin = int(rng.integers(2, 5))
                xs = [x] + [rnd_i8(rng, x.shape) for _ in range(nin - 1)]
                mult = [int(v) for v in rng.integers(-128, 128, nin)]
                rs, relu = int(rng.integers(0, 12)), bool(rng.integers(0, 2))
                want = O.eltwise_add_i8(xs, mult, [rs], relu)
                xts = [xt] + [ctx.from_nchw(v) for v in xs[1:]]
                yt = ctx.tensor(x.shape)
                tmp += xts[1:] + [yt]
                ctx.eltwise_add(xts, mult, rs, relu, yt)
            elif kind == "lut":
                table = rnd_i8(rng, 256)
                want = table[x.astype(np.uint8)]
                yt = ctx.tensor(x.shape)
                tmp.append(yt)
                ctx.lut(xt, yt, table)
            elif kind == "leaky":
                rp, mp, rn, mn = (int(rng.integers(0, 9)), int(rng.integers(1, 128)), int(rng.integers(0, 9)),
                                  int(rng.integers(1, 128)))
                want = O.leaky_relu_i8(x, rp, mp, rn, mn)
                yt = ctx.tensor(x.shape)
                tmp.append(yt)
                ctx.leaky_relu(xt, yt, rp, mp, rn, mn)
            elif kind == "up":
                sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
                want = O.upsample_i8(x, sh, sw)
                yt = ctx.tensor(want.shape)
                tmp.append(yt)
                ctx.upsample(xt, yt, sh, sw)
            else:
                axis, nin, xs = int(rng.integers(0, 4)), int(rng.integers(2, 5)), [x]
                for _ in range(nin - 1):
                    shp = list(x.shape)
                    shp[axis] = int(rng.integers(1, 40))
                    xs.append(rnd_i8(rng, shp))
                rs = mult = None
                relu = False
                if rng.integers(0, 2):
                    rs = [int(v) for v in rng.integers(0, 8, nin)]
                    mult = [int(v) for v in rng.integers(1, 128, nin)]
                    relu = bool(rng.integers(0, 2))
                want = O.concat_i8(xs, axis, rs, mult, relu)
                xts = [xt] + [ctx.from_nchw(v) for v in xs[1:]]
                yt = ctx.tensor(want.shape)
                tmp += xts[1:] + [yt]
                ctx.concat(xts, axis, yt, rs, mult, relu)
            assert np.array_equal(ctx.to_nchw(yt), want), (it, kind, x.shape, want.shape)
            assert not ctx.raw(yt)[..., want.shape[1]:].any(), (it, kind)
            seen[kind] = seen.get(kind, 0) + 1
        finally:
            for t in tmp:
                t.free()
    assert len(seen) == 7 and min(seen.values()) > 50, seen
