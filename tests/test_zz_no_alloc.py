"""The allocation-free FullyConnected entry point (tpuhip_fc_i8_noalloc) through the C ABI: its
output must equal that of tpuhip_fc_i8 -- one launch with the partial sums in LDS for the
first, long-K layer; for the second the same split-K kernels with a scratch buffer the library
allocates -- byte for byte, on two calls in a row, the second on a smaller input (the static
scratch keeps the first call's partial sums)."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_helpers import f2i32
from tpu_compiler_amd import capi

pytestmark = pytest.mark.gpu


def _fc_case(ctx, rng, m, k, n, relu):
    x = rng.integers(-128, 128, (m, k), dtype=np.int64).astype(np.int8)
    w = np.clip(np.rint(rng.normal(0, 20, (n, k))), -127, 127).astype(np.int8)
    bias = rng.integers(-3000, 3000, n).astype(np.float32)
    mult, rsh = np.float32((1 << 30) + 128 * 12345), np.float32(9)
    want = O.fc_i8(x, w, bias, [rsh], [mult], 1, m, k, n, relu)[0]
    xt = ctx.from_nchw(x.reshape(m, k, 1, 1))
    wh = ctx.fc_prepack(m, k, n, xt.cs, capi.channel_stride(n), relu, w, f2i32(bias), f2i32([mult])[0], f2i32([rsh])[0])
    return xt, wh, want


def test_fc_noalloc_equals_fc_on_two_calls_in_a_row():
    ctx = capi.Context(0)
    rng = np.random.default_rng(77)
    for m, k, n, relu in ((32, 2048, 1000, False), (5, 300, 37, True)):     # the second call is the smaller one
        xt, wh, want = _fc_case(ctx, rng, m, k, n, relu)
        y_ws, y_static = ctx.tensor((m, n, 1, 1)), ctx.tensor((m, n, 1, 1))
        for t in (y_ws, y_static):
            ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, 0x55, t.nbytes))
        ctx.fc(wh, xt, y_ws)
        ctx.fc(wh, xt, y_static, noalloc=True)
        a, b = ctx.to_nchw(y_ws).reshape(m, n), ctx.to_nchw(y_static).reshape(m, n)
        assert np.array_equal(a, want), "the workspace path differs from the oracle"
        assert np.array_equal(b, a), "the static-scratch path differs from the workspace path"
        assert np.array_equal(ctx.raw(y_static), ctx.raw(y_ws))             # pad channels too
        # once more on the same buffers
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, y_static.ptr, 0x55, y_static.nbytes))
        ctx.fc(wh, xt, y_static, noalloc=True)
        assert np.array_equal(ctx.raw(y_static), ctx.raw(y_ws))
        ctx.conv_weights_destroy(wh)
        for t in (xt, y_ws, y_static):
            t.free()
    ctx.close()


def test_fc_noalloc_leaves_the_free_device_memory_unchanged():
    """after a first call (which loads the code object) further calls take no device memory: the
    runtime's free-memory figure is the same before and after"""
    ctx = capi.Context(0)
    rng = np.random.default_rng(78)
    xt, wh, want = _fc_case(ctx, rng, 32, 512, 200, True)
    yt = ctx.tensor((32, 200, 1, 1))
    ctx.fc(wh, xt, yt, noalloc=True)
    ctx.sync()
    before = ctx.mem_info()[0]
    for _ in range(3):
        ctx.fc(wh, xt, yt, noalloc=True)
    ctx.sync()
    assert ctx.mem_info()[0] == before
    assert np.array_equal(ctx.to_nchw(yt).reshape(32, 200), want)
    ctx.conv_weights_destroy(wh)
    ctx.close()


def test_fc_noalloc_refuses_a_call_that_would_overlap_another_context():
    """two contexts (two streams) share the GPU's static scratch: while the first one's stream still has
    work in flight the second one's call is refused; once the first has drained it goes through"""
    a, b = capi.Context(0), capi.Context(0)
    rng = np.random.default_rng(79)
    xa, wa, want_a = _fc_case(a, rng, 32, 512, 200, True)
    xb, wb, want_b = _fc_case(b, rng, 8, 256, 64, False)
    ya, yb = a.tensor((32, 200, 1, 1)), b.tensor((8, 64, 1, 1))
    n = 256 << 20
    src, dst = a.malloc(n), a.malloc(n)
    a._ck(a.lib.tpuhip_memset(a.h, src, 1, n))
    a.sync()
    for _ in range(100):                 # some milliseconds of queued work on a's stream
        a._ck(a.lib.tpuhip_relu_i8(a.h, src, dst, n))
    a.fc(wa, xa, ya, noalloc=True)
    with pytest.raises(capi.TpuHipError, match="still in flight"):
        b.fc(wb, xb, yb, noalloc=True)
    a.sync()
    b.fc(wb, xb, yb, noalloc=True)
    assert np.array_equal(a.to_nchw(ya).reshape(32, 200), want_a)
    assert np.array_equal(b.to_nchw(yb).reshape(8, 64), want_b)
    a.free(src)
    a.free(dst)
    a.conv_weights_destroy(wa)
    b.conv_weights_destroy(wb)
    a.close()
    b.close()


def test_fc_noalloc_refuses_what_does_not_fit():
    ctx = capi.Context(0)
    rng = np.random.default_rng(5)
    # 256 rows x 8192 channels: 8 x 256 = 2048 blocks of 32 x 32 outputs, more than the split-K kernels take
    xt, wh, want = _fc_case(ctx, rng, 256, 128, 8192, False)
    yt = ctx.tensor((256, 8192, 1, 1))
    with pytest.raises(capi.TpuHipError, match="blocks of 32 x 32"):
        ctx.fc(wh, xt, yt, noalloc=True)
    ctx.fc(wh, xt, yt)           # the allocating entry point takes it (on the conv path)
    assert np.array_equal(ctx.to_nchw(yt).reshape(256, 8192), want)
    ctx.conv_weights_destroy(wh)
    # a conv is not a FullyConnected
    from gpu_helpers import conv_desc
    d = conv_desc((1, 32, 4, 4), (32, 32, 1, 1))
    wc = ctx.conv_prepack(d, np.ones((32, 32, 1, 1), np.int8), None, np.full(32, 1 << 30, np.int32), np.full(32, 8, np.int32))
    with pytest.raises(capi.TpuHipError, match="FullyConnected"):
        ctx._ck(ctx.lib.tpuhip_fc_i8_noalloc(ctx.h, wc, xt.ptr, yt.ptr))
    ctx.conv_weights_destroy(wc)
    ctx.close()
