"""Stand-alone bandwidth of the HBM-bound op kernels: `python -m tpu_compiler_amd.op_bench`.

One launch of each op through the C ABI at the largest shape it takes in the benchmark graphs
(ResNet-50 at batch 32, MobileNetV2 at batch 64, YOLOv3 at 608x608 and batch 8), timed with HIP
events over a run of launches on the context's stream.  Algorithmic bytes = every int8 input once
+ the output once, logical channels only.  A dependent launch costs about 2.4 us on this part
before any byte moves, which is what the small shapes show.  One table row per op on stdout.

A call from Python takes 3-5 us to enqueue, as long as the smaller kernels run, and a pause of the
interpreter (a garbage collection) lands in the middle of a run of launches now and then.  So that
the events bracket kernels running back to back and not the host's pace, the stream is first kept
busy with launches over a large buffer for longer than the host needs to enqueue the whole run;
"host" in the table is the enqueue time per launch, for comparison.
"""
import argparse
import gc
import math
import sys
import time

import numpy as np

from . import capi

PEAK_HBM_TBS = 8.0   # MI355X HBM3E


def _pool(x_shape, k, s, pads):
    n, c, ih, iw = x_shape
    pt, pb, pl, pr = pads
    oh, ow = (ih + pt + pb - k[0]) // s[0] + 1, (iw + pl + pr - k[1]) // s[1] + 1
    cs = capi.channel_stride(c)
    return capi.PoolDesc(n, c, ih, iw, oh, ow, k[0], k[1], s[0], s[1], pt, pb, pl, pr, cs, cs), (n, c, oh, ow)


def _depthwise(x_shape, stride):
    """3x3 depthwise conv with pad 1 and ReLU, as in the MobileNetV2 blocks"""
    n, c, ih, iw = x_shape
    oh, ow = (ih + 2 - 3) // stride + 1, (iw + 2 - 3) // stride + 1
    cs = capi.channel_stride(c)
    d = capi.ConvDesc(n, c, ih, iw, c, oh, ow, c, 3, 3, stride, stride, 1, 1, 1, 1, 1, 1, 0, 0, 1, 1, cs, cs, 0, 0)
    return d, (n, c, oh, ow)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--iters", type=int, default=20)
    args = ap.parse_args(argv)

    ctx = capi.Context(0)
    e0, e1 = ctx.event(), ctx.event()
    live = []

    def tensor(shape, fill=3):
        t = ctx.tensor(shape)
        ctx._ck(ctx.lib.tpuhip_memset(ctx.h, t.ptr, fill, t.nbytes))
        live.append(t)
        return t

    def release():
        ctx.sync()
        while live:
            live.pop().free()

    def logical(*ts):
        return sum(int(np.prod(t.shape)) for t in ts)

    def run_of(fn, n):
        """enqueues e0, n launches, e1; returns (GPU us, host enqueue us) per launch"""
        h0 = time.perf_counter()
        ctx.record(e0)
        for _ in range(n):
            fn()
        ctx.record(e1)
        h1 = time.perf_counter()
        ctx.sync()
        return ctx.elapsed_ms(e0, e1) / n * 1e3, (h1 - h0) / n * 1e6

    # what keeps the stream busy while the host enqueues: a read + write pass over 256 MiB
    busy_bytes = 256 << 20
    busy_src, busy_dst = ctx.malloc(busy_bytes), ctx.malloc(busy_bytes)
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, busy_src, 1, busy_bytes))

    def busy():
        ctx._ck(ctx.lib.tpuhip_relu_i8(ctx.h, busy_src, busy_dst, busy_bytes))

    for _ in range(3):
        busy()
    ctx.sync()
    busy_us = run_of(busy, 10)[0]

    def row(name, fn, nbytes):
        for _ in range(3):
            fn()
        ctx.sync()
        host_us = run_of(fn, args.iters)[1]
        # twice the time the host needs for the run, so that every launch is queued before the first one starts
        for _ in range(int(math.ceil(2.0 * (args.iters + 2) * host_us / busy_us)) + 1):
            busy()
        us, host_us = run_of(fn, args.iters)
        tbs = nbytes / us / 1e6
        print("%-52s %7.1f us (host %4.1f) %7.1f MB %6.2f TB/s %5.1f %% of %g TB/s" % (
            name, us, host_us, nbytes / 1e6, tbs, tbs / PEAK_HBM_TBS * 100, PEAK_HBM_TBS), flush=True)

    gc.disable()
    print("stream kept busy by passes that read 256 MiB and write 256 MiB, %.1f us each" % busy_us, flush=True)
    print("%-52s %10s %11s %10s %11s %s" % ("op, shape", "time", "", "bytes", "achieved", "of peak"), flush=True)

    # ResNet-50, batch 32: the res2 shortcut add and what shares its shape
    a, b, y = tensor((32, 256, 56, 56)), tensor((32, 256, 56, 56), 5), tensor((32, 256, 56, 56))
    row("eltwise_add 32x256x56x56 (resnet50)", lambda: ctx.eltwise_add([a, b], [50, 60], 7, True, y), logical(a, b, y))
    row("relu, same shape", lambda: ctx.relu(a, y), logical(a, y))
    table = np.arange(256).astype(np.int8)
    row("lut, same shape", lambda: ctx.lut(a, y, table), logical(a, y))
    row("eltwise max, same shape", lambda: ctx.binary(capi.BIN_MAX, a, b, y, m0=3, m1=2, rshift=1), logical(a, b, y))
    g = tensor((32, 256, 1, 1))
    row("broadcast_mul by 32x256x1x1", lambda: ctx.binary(capi.BIN_MUL, a, g, y, multiplier=1 << 30, rshift=5),
        logical(a, g, y))
    release()

    x = tensor((32, 64, 112, 112))
    d, y_shape = _pool(x.shape, (3, 3), (2, 2), (0, 1, 0, 1))
    y = tensor(y_shape)
    row("pool_max 3x3 s2 32x64x112x112 (resnet50)", lambda: ctx.pool_max(d, x, y), logical(x, y))
    release()
    x = tensor((32, 2048, 7, 7))
    d, y_shape = _pool(x.shape, (7, 7), (1, 1), (0, 0, 0, 0))
    y = tensor(y_shape)
    row("pool_avg global 32x2048x7x7 (resnet50)", lambda: ctx.pool_avg(d, x, y, 2, 7), logical(x, y))
    release()

    # YOLOv3, 608x608, batch 8
    a, y = tensor((8, 32, 608, 608)), tensor((8, 32, 608, 608))
    row("leaky_relu 8x32x608x608 (yolov3)", lambda: ctx.leaky_relu(a, y, 0, 0, 5, 3), logical(a, y))
    release()
    x, y = tensor((8, 128, 38, 38)), tensor((8, 128, 76, 76))
    row("upsample 2x 8x128x38x38 (yolov3)", lambda: ctx.upsample(x, y, 2, 2), logical(x, y))
    z, o = tensor((8, 256, 76, 76)), tensor((8, 384, 76, 76))
    row("concat 8x(128+256)x76x76 (yolov3)", lambda: ctx.concat([y, z], 1, o), logical(y, z, o))
    release()

    # depthwise 3x3: the two-layer block and the two largest MobileNetV2 layers
    for shape, stride, tag in (((8, 256, 56, 56), 1, "dw + pw block"), ((64, 96, 112, 112), 2, "mobilenetv2"),
                               ((64, 144, 56, 56), 1, "mobilenetv2")):
        d, y_shape = _depthwise(shape, stride)
        x, y = tensor(shape), tensor(y_shape)
        c = shape[1]
        w = ctx.conv_prepack(d, np.ones((c, 1, 3, 3), np.int8), np.zeros(c, np.int32),
                             np.full(c, 1 << 30, np.int32), np.full(c, 5, np.int32))
        row("depthwise 3x3 s%d %s (%s)" % (stride, "x".join(map(str, shape)), tag),
            lambda: ctx.conv(w, x, y), logical(x, y))
        ctx.sync()
        ctx.conv_weights_destroy(w)
        release()

    x, p = tensor((8, 256, 56, 56)), tensor((8, 56, 56, 256))
    row("permute to order 0,2,3,1 of 8x256x56x56", lambda: ctx.move(capi.MOVE_PERMUTE, x, p, [0, 2, 3, 1]),
        logical(x, p))
    release()
    ctx.free(busy_src)
    ctx.free(busy_dst)
    ctx.close()
    gc.enable()
    return 0


if __name__ == "__main__":
    sys.exit(main())
