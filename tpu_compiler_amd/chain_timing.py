"""Times the launches that run two convolutions as one (tpuhip_conv2d_chain_*) against the two launches
they replace, on the layer pairs of the benchmark networks:

    python -m tpu_compiler_amd.chain_timing [--batch-resnet 32] [--batch-mobilenet 64]

  * pointwise -> pointwise (ResNet-50: the 1x1 expansion + residual add closing a bottleneck block and
    the 1x1 reduction opening the next);
  * depthwise -> pointwise (MobileNetV2: the depthwise conv and the 1x1 projection of an
    inverted-residual block, with the block's residual add where it has one);
  * pointwise -> depthwise -> pointwise (the whole inverted-residual block).

Random weights and inputs; both forms write the same bytes (checked).  HIP events around 20 launches."""
import argparse

import numpy as np

from . import capi


def _desc(x_shape, oc, k, g=1, stride=1, pad=0, relu=False):
    n, ic, ih, iw = x_shape
    oh = (ih + 2 * pad - k) // stride + 1
    ow = (iw + 2 * pad - k) // stride + 1
    return capi.ConvDesc(n, ic, ih, iw, oc, oh, ow, g, k, k, stride, stride, pad, pad, pad, pad, 1, 1, 0, 0,
                         int(relu), 1, capi.channel_stride(ic), capi.channel_stride(oc), 0, 0)


def _params(rng, oc):
    bias = rng.integers(-1000, 1000, oc).astype(np.int32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.int32)
    rsh = rng.integers(8, 12, oc).astype(np.int32)
    return bias, mult, rsh


def _weights(rng, shape, sigma):
    return np.clip(np.rint(rng.normal(0, sigma, shape)), -127, 127).astype(np.int8)


def _time(ctx, fn, iters=20):
    for _ in range(3):
        fn()
    ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0)
    for _ in range(iters):
        fn()
    ctx.record(e1)
    return ctx.elapsed_ms(e0, e1) * 1e3 / iters


def _fill(ctx, rng, t):
    ctx.upload(t.ptr, rng.integers(-128, 128, t.nbytes, dtype=np.int64).astype(np.int8))


def _bytes(ctx, t):
    return ctx.download(t.ptr, (t.nbytes,), np.int8).copy()


def pointwise_pair(ctx, rng, n, ic, oc1, oc2, hw):
    """expansion ic -> oc1 + add + ReLU, reduction oc1 -> oc2 + ReLU"""
    wa, wb = _weights(rng, (oc1, ic, 1, 1), 20), _weights(rng, (oc2, oc1, 1, 1), 20)
    pa, pb = _params(rng, oc1), _params(rng, oc2)
    xs, ms = (n, ic, hw, hw), (n, oc1, hw, hw)
    da, db = _desc(xs, oc1, 1), _desc(ms, oc2, 1, relu=True)
    xt, ot, zt, z2 = ctx.tensor(xs), ctx.tensor(ms), ctx.tensor(ms), ctx.tensor(ms)
    y1, y2 = ctx.tensor((n, oc2, hw, hw)), ctx.tensor((n, oc2, hw, hw))
    _fill(ctx, rng, xt)
    _fill(ctx, rng, ot)
    wha, whb = ctx.conv_prepack(da, wa, *pa), ctx.conv_prepack(db, wb, *pb)
    ch = ctx.conv_chain_prepack(da, db, (wa, *pa), (wb, *pb))

    def separate():
        ctx.conv_add(wha, xt, None, ot, zt, 61, 47, 6, True)
        ctx.conv(whb, zt, y1)

    def chained():
        ctx.conv_chain(ch, xt, y2, None, (ot, z2, 61, 47, 6, True))

    separate()                                     # the tile choice by timing happens on first use
    ts, tc = _time(ctx, separate), _time(ctx, chained)
    same = np.array_equal(_bytes(ctx, y1), _bytes(ctx, y2)) and np.array_equal(_bytes(ctx, zt), _bytes(ctx, z2))
    names = "%s + %s" % (ctx.conv_algo_name(wha), ctx.conv_algo_name(whb))
    for t in (xt, ot, zt, z2, y1, y2):
        t.free()
    return ts, tc, same, names, ctx.conv_chain_name(ch)


def depthwise_pair(ctx, rng, n, c, oc, hw, stride, add):
    """3x3 depthwise on c channels + ReLU, 1x1 projection c -> oc, residual add where the block has one"""
    wa, wb = _weights(rng, (c, 1, 3, 3), 30), _weights(rng, (oc, c, 1, 1), 20)
    pa, pb = _params(rng, c), _params(rng, oc)
    xs = (n, c, hw, hw)
    da = _desc(xs, c, 3, g=c, stride=stride, pad=1, relu=True)
    ms, ys = (n, c, da.oh, da.ow), (n, oc, da.oh, da.ow)
    db = _desc(ms, oc, 1)
    xt, mt, ot = ctx.tensor(xs), ctx.tensor(ms), ctx.tensor(ys)
    r1, r2 = ctx.tensor(ys), ctx.tensor(ys)
    _fill(ctx, rng, xt)
    _fill(ctx, rng, ot)
    wha, whb = ctx.conv_prepack(da, wa, *pa), ctx.conv_prepack(db, wb, *pb)
    ch = ctx.conv_chain_prepack(da, db, (wa, *pa), (wb, *pb))

    def separate():
        ctx.conv(wha, xt, mt)
        if add:
            ctx.conv_add(whb, mt, None, ot, r1, 64, 64, 7, False)
        else:
            ctx.conv(whb, mt, r1)

    def chained():
        if add:
            ctx.conv_chain_post(ch, xt, add_b=(ot, r2, 64, 64, 7, False))
        else:
            ctx.conv_chain_post(ch, xt, y_b=r2)

    separate()
    ts, tc = _time(ctx, separate), _time(ctx, chained)
    same = np.array_equal(_bytes(ctx, r1), _bytes(ctx, r2))
    names = "%s + %s" % (ctx.conv_algo_name(wha), ctx.conv_algo_name(whb))
    for t in (xt, mt, ot, r1, r2):
        t.free()
    return ts, tc, same, names, ctx.conv_chain_name(ch)


def inverted_residual(ctx, rng, n, cin, c, oc, hw, stride, add):
    """1x1 expansion cin -> c + ReLU, 3x3 depthwise + ReLU, 1x1 projection c -> oc, residual add where the
    block has one"""
    we, wa, wb = _weights(rng, (c, cin, 1, 1), 24), _weights(rng, (c, 1, 3, 3), 30), _weights(rng, (oc, c, 1, 1), 20)
    pe, pa, pb = _params(rng, c), _params(rng, c), _params(rng, oc)
    xs, es = (n, cin, hw, hw), (n, c, hw, hw)
    de = _desc(xs, c, 1, relu=True)
    da = _desc(es, c, 3, g=c, stride=stride, pad=1, relu=True)
    ms, ys = (n, c, da.oh, da.ow), (n, oc, da.oh, da.ow)
    db = _desc(ms, oc, 1)
    xt, et, mt, ot = ctx.tensor(xs), ctx.tensor(es), ctx.tensor(ms), ctx.tensor(ys)
    r1, r2 = ctx.tensor(ys), ctx.tensor(ys)
    _fill(ctx, rng, xt)
    _fill(ctx, rng, ot)
    whe, wha, whb = ctx.conv_prepack(de, we, *pe), ctx.conv_prepack(da, wa, *pa), ctx.conv_prepack(db, wb, *pb)
    ch = ctx.conv_chain3_prepack(de, da, db, (we, *pe), (wa, *pa), (wb, *pb))

    def separate():
        ctx.conv(whe, xt, et)
        ctx.conv(wha, et, mt)
        if add:
            ctx.conv_add(whb, mt, None, ot, r1, 64, 64, 7, False)
        else:
            ctx.conv(whb, mt, r1)

    def chained():
        if add:
            ctx.conv_chain3(ch, xt, None, (ot, r2, 64, 64, 7, False))
        else:
            ctx.conv_chain3(ch, xt, r2)

    separate()
    ts, tc = _time(ctx, separate), _time(ctx, chained)
    same = np.array_equal(_bytes(ctx, r1), _bytes(ctx, r2))
    names = "%s + %s + %s" % (ctx.conv_algo_name(whe), ctx.conv_algo_name(wha), ctx.conv_algo_name(whb))
    for t in (xt, et, mt, ot, r1, r2):
        t.free()
    return ts, tc, same, names, ctx.conv_chain_name(ch)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--batch-resnet", type=int, default=32)
    ap.add_argument("--batch-mobilenet", type=int, default=64)
    args = ap.parse_args()
    ctx = capi.Context(0)
    rng = np.random.default_rng(1)
    print("pointwise -> pointwise, batch %d: us for the two launches | the chain" % args.batch_resnet)
    for ic, oc1, oc2, hw in ((64, 256, 64, 56), (128, 512, 128, 28)):
        ts, tc, same, names, cname = pointwise_pair(ctx, rng, args.batch_resnet, ic, oc1, oc2, hw)
        print("  %3d -> %3d (+add) -> %3d at %2dx%-2d  %6.2f | %6.2f  %s | %s  %s"
              % (ic, oc1, oc2, hw, hw, ts, tc, names, cname, "same bytes" if same else "BYTES DIFFER"), flush=True)
    print("depthwise 3x3 -> pointwise, batch %d: us for the two launches | the chain" % args.batch_mobilenet)
    tot = [0.0, 0.0]
    for c, oc, hw, s, add in ((32, 16, 112, 1, False), (96, 24, 112, 2, False), (144, 24, 56, 1, True),
                              (144, 32, 56, 2, False), (192, 32, 28, 1, True), (192, 64, 28, 2, False),
                              (384, 64, 14, 1, True), (384, 96, 14, 1, False), (576, 96, 14, 1, True),
                              (576, 160, 14, 2, False), (960, 160, 7, 1, True), (960, 320, 7, 1, False)):
        ts, tc, same, names, cname = depthwise_pair(ctx, rng, args.batch_mobilenet, c, oc, hw, s, add)
        tot[0] += ts
        tot[1] += tc
        print("  %3d dw s%d%s -> %3d at %3dx%-3d  %6.2f | %6.2f  %s | %s  %s"
              % (c, s, " (+add)" if add else "       ", oc, hw, hw, ts, tc, names, cname,
                 "same bytes" if same else "BYTES DIFFER"), flush=True)
    print("  sum %.1f | %.1f" % tuple(tot))
    print("1x1 -> depthwise 3x3 -> 1x1, batch %d: us for the three launches | the chain" % args.batch_mobilenet)
    tot = [0.0, 0.0]
    for cin, c, oc, hw, s, add in ((16, 96, 24, 112, 2, False), (24, 144, 24, 56, 1, True), (24, 144, 32, 56, 2, False),
                                   (32, 192, 32, 28, 1, True), (32, 192, 64, 28, 2, False), (64, 384, 64, 14, 1, True),
                                   (64, 384, 96, 14, 1, False), (96, 576, 96, 14, 1, True), (96, 576, 160, 14, 2, False),
                                   (160, 960, 160, 7, 1, True), (160, 960, 320, 7, 1, False)):
        if not ctx.conv_can_chain3(_desc((args.batch_mobilenet, cin, hw, hw), c, 1, relu=True),
                                   _desc((args.batch_mobilenet, c, hw, hw), c, 3, g=c, stride=s, pad=1, relu=True),
                                   _desc((args.batch_mobilenet, c, (hw - 1) // s + 1, (hw - 1) // s + 1), oc, 1)):
            print("  %3d -> %3d dw s%d -> %3d at %3dx%-3d  not covered" % (cin, c, s, oc, hw, hw))
            continue
        ts, tc, same, names, cname = inverted_residual(ctx, rng, args.batch_mobilenet, cin, c, oc, hw, s, add)
        tot[0] += ts
        tot[1] += tc
        print("  %3d -> %3d dw s%d%s -> %3d at %3dx%-3d  %6.2f | %6.2f  %s | %s  %s"
              % (cin, c, s, " (+add)" if add else "       ", oc, hw, hw, ts, tc, names, cname,
                 "same bytes" if same else "BYTES DIFFER"), flush=True)
    print("  sum %.1f | %.1f" % tuple(tot))
    ctx.close()


if __name__ == "__main__":
    main()
