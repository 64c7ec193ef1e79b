"""GPU parity tests of the two-convs-in-one-launch entry point (tpuhip_conv2d_chain_*): pointwise conv A,
an optional EltwiseAdd on its result, pointwise conv B on the sum -- every tensor equal to the oracle's
three ops run one after the other."""
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


def rnd_params(rng, oc, rs_lo=8, rs_hi=20, bias_mag=4096):
    bias = rng.integers(-bias_mag, bias_mag + 1, oc).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
    rsh = rng.integers(rs_lo, rs_hi + 1, oc).astype(np.float32)
    return bias, rsh, mult


def oracle_pw(x, w, bias, rsh, mult, relu):
    d = O.make_conv_desc(x.shape, w.shape, 1, (1, 1), (0, 0, 0, 0), (1, 1), (0, 0), relu, True, None)
    return O.conv2d_i8(x, w, bias, rsh, mult, d)


# (ic, oc1, oc2): the channel triples the kernel variants cover
SHAPES = [(64, 256, 64), (48, 256, 64), (128, 512, 128), (80, 512, 128)]
# (n, h, w): pixel counts that end inside a 64-pixel tile, fill one exactly, and span many workgroups
PIXELS = [(1, 5, 7), (2, 8, 4), (3, 17, 13), (2, 56, 56)]


def run_chain(ctx, rng, ic, oc1, oc2, nhw, relu_a, relu_b, add, keep_a, keep_sum=True, rs_lo=8, rs_hi=20):
    n, h, w = nhw
    x = rnd_i8(rng, (n, ic, h, w))
    wa, wb = rnd_w(rng, (oc1, ic, 1, 1)), rnd_w(rng, (oc2, oc1, 1, 1), 12)
    pa, pb = rnd_params(rng, oc1, rs_lo, rs_hi), rnd_params(rng, oc2, rs_lo + 1, rs_hi)
    ya = oracle_pw(x, wa, *pa, relu_a)
    mid = ya
    if add:
        other = rnd_i8(rng, ya.shape)
        m_src, m_conv, rs, relu = add
        mid = O.eltwise_add_i8([other, ya], [m_src, m_conv], [rs], relu)
    yb = oracle_pw(mid, wb, *pb, relu_b)
    da = conv_desc(x.shape, wa.shape, do_relu=relu_a)
    db = conv_desc(ya.shape, wb.shape, do_relu=relu_b)
    assert ctx.conv_can_chain(da, db)
    ch = ctx.conv_chain_prepack(da, db, (wa, f2i32(pa[0]), f2i32(pa[2]), f2i32(pa[1])),
                                (wb, f2i32(pb[0]), f2i32(pb[2]), f2i32(pb[1])))
    xt = ctx.from_nchw(x)
    yat, zt, ybt = ctx.tensor(ya.shape), ctx.tensor(ya.shape), ctx.tensor(yb.shape)
    for t in (yat, zt, ybt):
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
    ot = ctx.from_nchw(other) if add else None
    ctx.conv_chain(ch, xt, ybt, yat if keep_a else None,
                   (ot, zt if keep_sum else None, m_src, m_conv, rs, relu) if add else None)
    assert np.array_equal(ctx.to_nchw(ybt), yb), "conv B"
    if keep_a:
        assert np.array_equal(ctx.to_nchw(yat), ya), "conv A"
    else:
        assert (ctx.raw(yat) == 0x55).all()
    if add and keep_sum:
        assert np.array_equal(ctx.to_nchw(zt), mid), "sum"
    else:
        assert (ctx.raw(zt) == 0x55).all()
    ctx.conv_chain_destroy(ch)
    for t in (xt, yat, zt, ybt) + ((ot,) if ot else ()):
        t.free()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("nhw", PIXELS)
def test_chain_with_add(ctx, shape, nhw):
    """the residual form: expansion (no ReLU) + add (ReLU) + reduction (ReLU); A's result not kept"""
    rng = np.random.default_rng(shape[0] * 7 + nhw[1])
    run_chain(ctx, rng, *shape, nhw, False, True, (61, 47, 6, True), False)


@pytest.mark.parametrize("shape", SHAPES[::2])
@pytest.mark.parametrize("relu_a,relu_b,add,keep_a,keep_sum", [
    (False, True, (61, 47, 6, True), True, True),       # every tensor kept
    (True, False, (-61, 47, 0, False), True, True),     # ReLU on A, none on B, add without shift or ReLU
    (False, True, (100, -128, 9, True), False, True),   # a shift beyond the packed-int16 form
    (True, True, None, True, True),                     # no add: B reads A's result
    (False, False, None, False, True),                  # ... which then is not written at all
    (False, True, (61, 47, 6, True), False, False),     # only B's result leaves the launch
])
def test_chain_forms(ctx, shape, relu_a, relu_b, add, keep_a, keep_sum):
    rng = np.random.default_rng(shape[1] + (17 if add else 3))
    run_chain(ctx, rng, *shape, (2, 9, 11), relu_a, relu_b, add, keep_a, keep_sum)


def test_chain_extreme_shifts(ctx):
    """right shifts 1 and 31, accumulators as large as 8-bit operands make them"""
    rng = np.random.default_rng(5)
    run_chain(ctx, rng, 64, 256, 64, (1, 6, 6), False, True, (61, 47, 6, True), True, rs_lo=1, rs_hi=31)


def test_chain_refuses_what_it_cannot_run(ctx):
    rng = np.random.default_rng(9)
    x = (1, 64, 4, 4)
    wa, wb = rnd_w(rng, (256, 64, 1, 1)), rnd_w(rng, (64, 256, 1, 1))
    da, db = conv_desc(x, wa.shape), conv_desc((1, 256, 4, 4), wb.shape)
    pa, pb = rnd_params(rng, 256), rnd_params(rng, 64)
    pa[1][3] = 0      # a right shift of 0: the overflow-free rounding needs at least 1
    with pytest.raises(capi.TpuHipError):
        ctx.conv_chain_prepack(da, db, (wa, f2i32(pa[0]), f2i32(pa[2]), f2i32(pa[1])),
                               (wb, f2i32(pb[0]), f2i32(pb[2]), f2i32(pb[1])))
    # a 3x3 first conv, a second conv that does not read the first one's channel count
    assert not ctx.conv_can_chain(conv_desc(x, (256, 64, 3, 3), pads=(1, 1, 1, 1)), db)
    assert not ctx.conv_can_chain(da, conv_desc((1, 128, 4, 4), (64, 128, 1, 1)))
