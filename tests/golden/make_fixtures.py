#!/usr/bin/env python3
"""Writes the committed fixtures of this directory.

The reference holds no input/output vectors for its INT8 interpreter path (its
regression flow compares against framework outputs it downloads), so the vectors
kept here are generated: small seeded quantized graphs, every tensor of which is
computed by the CPU oracle (tests/oracle_graph.py over oracle/tpu_oracle.c), whose
arithmetic is pinned separately by tests/test_oracle.py.

For every graph NAME three files are written:
  NAME.mlir          the graph in the TPU dialect's textual form
  NAME_weights.npz   its weight file (the name the .mlir records)
  NAME_io.npz        "<input name>" and every other tensor of the graph, as the
                     oracle computes it (int8 / uint8 / float32 as the tensor is)

tests/test_golden.py checks that the oracle still reproduces NAME_io.npz from a
rebuild of the graph, and that the HIP path, loading NAME.mlir through the C ABI,
produces the same tensors.

  python tests/golden/make_fixtures.py [--check]
"""
import argparse
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))                       # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))      # repository root

from tpu_compiler_amd import graphs, mlir_text  # noqa: E402

f32 = lambda *v: np.array(v, np.float32)  # noqa: E731


def mini_net():
    """3-channel stem, leaky relu, max pool, inverted residual (1x1 / depthwise / 1x1 + add),
    a strided branch brought back by upsample + concat, clip, global average, fc"""
    b = graphs.Builder("mini_net", graphs.BASE_SEED + 301, 2, (5, 14))
    x = b.input("input", 3, 40, 40)
    y = b.conv("stem", x, 16, 3, stride=2, relu=False)
    y = b.leaky("stem_leaky", y)
    p = b.pool_max("pool", y, 3, 2, (0, 1, 0, 1))
    e = b.conv("expand", p, 48, 1, relu=True)
    d = b.conv("dw", e, 48, 3, groups=48, relu=True)
    r = b.conv("project", d, 16, 1, relu=False)
    a = b.add("res", [r, p], relu=True)
    s = b.conv("down", a, 32, 3, stride=2, pads=(1, 0, 1, 0), relu=True)
    u = b.upsample("up", s, 2)
    c = b.concat("cat", [u, a])
    h = b.conv("head", c, 40, (1, 3), relu=True, pads=(0, 0, 1, 1))
    h = b.clip("head_clip", h, 0, 90)
    gp = b.global_avg("gap", h)
    fl = b.reshape("flat", gp, (2, 40))
    out = b.fc("fc", fl, 10)
    return b.finish([out]), None


def se_block():
    """prelu, eltwise max / min / mul, global average, broadcast mul / add / sub, and a
    table-lookup activation"""
    b = graphs.Builder("se_block", graphs.BASE_SEED + 302, 2, (6, 12))
    x = b.input("input", 8, 10, 9)
    c1 = b.conv("c1", x, 24, 3, relu=True)
    c2 = b.conv("c2", x, 24, 3, relu=False)
    g = b.g
    shp = g.by_name[c1].shape

    def binop(t, name, srcs, mult, rshift, relu=0):
        g.add(graphs.Op(t, name, srcs, shp, dict(do_relu=relu),
                        dict(rshift=f32(rshift), multiplier=f32(*mult)), "RSHIFT_AND_M_I8"))
        return name

    slope = (np.arange(shp[1]) % 23 - 7).astype(np.float32)
    g.add(graphs.Op("tpu.prelu", "pr", [c2], shp, {},
                    dict(slope=slope, rshift_pos=f32(1), multiplier_pos=f32(3), rshift_neg=f32(3)),
                    "RSHIFT_AND_M_I8"))
    mx = binop("tpu.eltwise_max", "mx", [c1, c2], (3, 2), 1)
    mn = binop("tpu.eltwise_min", "mn", [c1, "pr"], (1, 1), 0, relu=1)
    ml = binop("tpu.eltwise_mul", "ml", [mx, mn], (1518500250,), 6)
    g.add(graphs.Op("tpu.pool_avg_2d", "gap", [ml], (shp[0], shp[1], 1, 1),
                    dict(kernel_h=shp[2], kernel_w=shp[3], stride_h=1, stride_w=1, padding_t=0,
                         padding_b=0, padding_l=0, padding_r=0, do_relu=0),
                    dict(rshift=f32(7), multiplier=f32(2)), "RSHIFT_AND_M_I8"))
    gate = binop("tpu.broadcast_mul", "gate", [mx, "gap"], (1 << 30,), 5)
    ba = binop("tpu.broadcast_add", "badd", [gate, "gap"], (2, 3), 2, relu=1)
    bs = binop("tpu.broadcast_sub", "bsub", ["gap", ba], (9, 5), 1)
    table = np.clip(np.rint(127 / (1 + np.exp(-np.arange(-128, 128) / 16.0))), -128, 127)
    table = np.roll(table, 128).astype(np.float32)      # entry i <-> two's-complement byte i
    g.add(graphs.Op("tpu.sigmoid", "sig", [bs], shp, {}, {"table": table}, "LUT_INT8"))
    g.outputs = ["sig"]
    return g, None


def movers():
    """pad (constant and edge), crop, permute, reorg, pixel shuffle, tile, reverse, channel
    shuffle, average pool with padding, relu"""
    b = graphs.Builder("movers", graphs.BASE_SEED + 303, 2, (6, 12))
    x = b.input("input", 6, 8, 6)
    c1 = b.conv("c1", x, 36, 3, relu=False)
    g = b.g
    n = 2

    def mv(t, name, src, shape, **attrs):
        g.add(graphs.Op(t, name, [src], shape, attrs))
        return name

    p = mv("tpu.pad", "pad", c1, (n, 36, 11, 9), pads0=0, pads1=0, pads2=1, pads3=2, pads4=0,
           pads5=0, pads6=2, pads7=1)
    mv("tpu.pad", "pad_edge", c1, (n, 36, 10, 8), mode_edge=1, pads0=0, pads1=0, pads2=1, pads3=1,
       pads4=0, pads5=0, pads6=1, pads7=1)
    cr = mv("tpu.crop", "crop", p, (n, 20, 8, 6), crop_offset0=0, crop_offset1=4, crop_offset2=1,
            crop_offset3=2)
    mv("tpu.permute", "perm", cr, (n, 8, 6, 20), order0=0, order1=2, order2=3, order3=1)
    ro = mv("tpu.reorg", "reorg", c1, (n, 144, 4, 3), stride=2)
    d2s = mv("tpu.pixelshuffle", "d2s", ro, (n, 36, 8, 6), upscale_factor=2, mode_dcr=1)
    tl = mv("tpu.tile", "tile", d2s, (n, 36, 8, 18), axis=3, tiles=3)
    rv = mv("tpu.reverse", "rev", tl, (n, 36, 8, 18), axis=2)
    mv("tpu.shuffle_channel", "shuf", rv, (n, 36, 8, 18), group=4)
    mv("tpu.relu", "relu", c1, (n, 36, 8, 6))
    g.add(graphs.Op("tpu.pool_avg_2d", "avg", [c1], (n, 36, 4, 3),
                    dict(kernel_h=3, kernel_w=3, stride_h=2, stride_w=2, padding_t=1, padding_b=0,
                         padding_l=1, padding_r=0, do_relu=0, count_include_pad=0),
                    dict(rshift=f32(9), multiplier=f32(57)), "RSHIFT_AND_M_I8"))
    g.outputs = ["perm", "pad_edge", "shuf", "relu", "avg"]
    return g, None


def uint8_front():
    """uint8 image -> per-channel 256-entry tables (ScaleLut) -> conv"""
    rng = np.random.default_rng(306)
    b = graphs.Builder("uint8_front", graphs.BASE_SEED + 304, 2, (6, 12))
    x8 = b.input("x8", 3, 12, 10)                # calibrates the conv; replaced below
    c1 = b.conv("c1", x8, 24, 3, relu=True)
    g = b.g
    shape = g.by_name["x8"].shape
    img = rng.integers(0, 256, shape).astype(np.uint8)
    img.flat[:4] = [0, 127, 128, 255]
    idx = np.arange(256)
    scale, bias = np.array([0.9, 1.0, 0.4]), np.array([-110.0, -128.0, 11.0])
    table = np.clip(np.floor(idx[None] * scale[:, None] + bias[:, None] + 0.5), -128, 127)
    fin = graphs.Op("tpu.input", "input", [], shape)
    fin.quant = "UINT8"
    fin.data = img
    sl = graphs.Op("tpu.scale_lut", "x8", ["input"], shape, {},
                   dict(table=table.astype(np.float32).reshape(-1)))
    g.ops[0:1] = [fin, sl]
    g.by_name["input"] = fin
    g.by_name["x8"] = sl
    g.outputs = [c1]
    return g, img


def fp32_edges():
    """fp32 input -> quantize -> conv -> transposed conv -> dequantize"""
    rng = np.random.default_rng(305)
    b = graphs.Builder("fp32_edges", graphs.BASE_SEED + 305, 2, (6, 12))
    x8 = b.input("x8", 12, 7, 6)                 # calibrates the conv; replaced below
    c1 = b.conv("c1", x8, 16, 3, relu=True)
    g = b.g
    shape = g.by_name["x8"].shape
    xf = rng.normal(0, 1.2, shape).astype(np.float32)
    xf.flat[:8] = [0.5 / 31.75, -0.5 / 31.75, 1.5 / 31.75, 4.1, -4.1, 100.0, -100.0, 0.0]
    fin = graphs.Op("tpu.input", "input", [], shape)
    fin.quant = "NONE"
    fin.data = xf
    q = graphs.Op("tpu.quant", "x8", ["input"], shape, dict(scale=31.75))
    g.ops[0:1] = [fin, q]
    g.by_name["input"] = fin
    g.by_name["x8"] = q
    oc, k = 20, 3
    w = np.clip(np.rint(rng.normal(0, 30, (oc, 16, k, k))), -127, 127).astype(np.float32)
    g.add(graphs.Op("tpu.deconv_2d", "up", [c1], (2, oc, 14, 12),
                    dict(kernel_h=k, kernel_w=k, stride_h=2, stride_w=2, padding_t=1, padding_b=1,
                         padding_l=1, padding_r=1, dilation_h=1, dilation_w=1, group=1, with_bias=1,
                         do_relu=0),
                    dict(filter=w.ravel(), bias=rng.integers(-2000, 2000, oc).astype(np.float32),
                         rshift=rng.integers(8, 12, oc).astype(np.float32),
                         multiplier=(rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)),
                    "RSHIFT_AND_M_I32"))
    dq = graphs.Op("tpu.quant", "out", ["up"], (2, oc, 14, 12), dict(scale=0.0207))
    dq.quant = "NONE"
    g.add(dq)
    g.outputs = ["out"]
    return g, xf


GRAPHS = [mini_net, se_block, movers, uint8_front, fp32_edges]


def build(fn):
    """-> (graph, input array as the graph's input tensor holds it)"""
    g, x = fn()
    return g, (g.input_op().data if x is None else x)


def expected(g, x):
    """every tensor of the graph from the oracle, shaped as the graph declares it"""
    import oracle_graph
    want = oracle_graph.run(g)
    return {op.name: np.ascontiguousarray(want[op.name]).reshape(op.shape) for op in g.ops}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--check", action="store_true", help="compare with the files present; write nothing")
    args = ap.parse_args()
    bad = 0
    for fn in GRAPHS:
        g, x = build(fn)
        want = expected(g, x)
        io_path = os.path.join(HERE, g.name + "_io.npz")
        if args.check:
            with np.load(io_path) as z:
                same = sorted(z.files) == sorted(want) and all(
                    z[k].dtype == want[k].dtype and np.array_equal(z[k], want[k]) for k in want)
            print("%-12s %s" % (g.name, "same" if same else "DIFFERS"))
            bad += not same
            continue
        mlir_text.write_mlir(g, os.path.join(HERE, g.name + ".mlir"))
        np.savez_compressed(io_path, **want)
        size = sum(os.path.getsize(os.path.join(HERE, g.name + s)) for s in (".mlir", "_weights.npz", "_io.npz"))
        print("%-12s %2d ops, %d tensors, %d KiB" % (g.name, len(g.ops), len(want), size // 1024))
    sys.exit(1 if bad else 0)


if __name__ == "__main__":
    main()
