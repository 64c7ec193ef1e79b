"""Quantized TPU-dialect graphs for the five benchmark configurations.

A graph is what the reference's quantization passes hand to tpuc-interpreter:
a list of TPU-level ops in program order, every weight-like operand a float32
array holding integers (filter, int32 bias, per-channel rshift and multiplier:
lib/Dialect/TPU/Quantization/QuantizeInt8.cpp:56-166).  The operand order of
each op follows the reference's kernels (core/conv.cpp:20-36,
core/eltwise.cpp:12-23, core/pooling.cpp:72-82, core/activation.cpp:113-121,
core/concat.cpp:13-17, core/fullyconnected.cpp:17-29).

Weights are random (seeded, integer-only generator); rshift values are chosen by
a calibration pass over one image, the way the reference derives them from
calibration thresholds, so that activations neither die out nor saturate as
they travel through 50+ layers.  The calibration arithmetic below serves graph
construction only; it never produces a result handed to a caller.
"""
import math

import numpy as np

from . import synth

TARGET_RMS = 40.0


class Op:
    def __init__(self, type_, name, inputs, shape, attrs=None, weights=None, param_type="NONE"):
        self.type = type_
        self.name = name
        self.inputs = list(inputs)
        self.shape = tuple(int(v) for v in shape)
        self.attrs = dict(attrs or {})
        self.weights = dict(weights or {})     # role -> float32 array (float-stored integers)
        self.quant = "INT8"
        self.param_type = param_type

    def __repr__(self):
        return "Op(%s %s %s)" % (self.type, self.name, self.shape)


class Graph:
    def __init__(self, name, seed):
        self.name = name
        self.seed = seed
        self.ops = []
        self.by_name = {}
        self.outputs = []
        self.stats = {}        # op name -> calibration statistics (zero / saturation fractions)
        self.macs = 0          # multiply-accumulates per run of the whole batch (conv + fc)

    def add(self, op):
        assert op.name not in self.by_name, op.name
        self.ops.append(op)
        self.by_name[op.name] = op
        return op

    def input_op(self):
        return self.ops[0]

    def conv_ops(self):
        return [o for o in self.ops if o.type in ("tpu.conv_2d", "tpu.fully_connected")]


# ---------------------------------------------------------------------------
# calibration arithmetic (graph construction only)
# ---------------------------------------------------------------------------

def _qdm(v, mult, rshift):
    """SaturatingRoundingDoublingHighMul + RoundingDivideByPOT + saturate, on int64 arrays
    (lib/Dialect/TPU/Quantization/QuantizationArithmetic.cpp:487-539)."""
    x = (v * mult + (1 << 30)) >> 31
    mask = (np.int64(1) << rshift) - 1
    rem = x & mask
    thr = (mask >> 1) + (x < 0)
    return np.clip((x >> rshift) + (rem > thr), -128, 127)


def _half_up_shift(v, r):
    return (v + ((np.int64(1) << r) >> 1)) >> r


def _conv_acc(x, w, stride, pads, dil, groups):
    import torch
    import torch.nn.functional as F
    xt = torch.from_numpy(x.astype(np.float32))
    pt, pb, pl, pr = pads
    if (pt, pl) != (pb, pr):
        xt = F.pad(xt, (pl, pr, pt, pb))
        padding = 0
    else:
        padding = (pt, pl)
    y = F.conv2d(xt, torch.from_numpy(w.astype(np.float32)), None, stride, padding, dil, groups)
    return np.rint(y.numpy()).astype(np.int64)


def _rms(a):
    a = a.astype(np.float64)
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


def _record(g, name, y):
    g.stats[name] = {
        "zero_frac": float(np.mean(y == 0)),
        "sat_frac": float(np.mean((y == 127) | (y == -128))),
        "rms": _rms(y),
    }


# ---------------------------------------------------------------------------
# builder
# ---------------------------------------------------------------------------

class Builder:
    """Appends ops to a graph while carrying one calibration image through it."""

    def __init__(self, name, seed, batch, rshift_range):
        self.g = Graph(name, seed)
        self.batch = batch
        self.rs_lo, self.rs_hi = rshift_range
        self.layer = 0
        self.cal = {}      # tensor name -> int64 NCHW calibration activation (batch 1)

    def _stream(self, kind):
        return (self.layer << 8) | kind

    def _out_hw(self, ih, iw, k, s, pads, d=(1, 1)):
        oh = (ih + pads[0] + pads[1] - (d[0] * (k[0] - 1) + 1)) // s[0] + 1
        ow = (iw + pads[2] + pads[3] - (d[1] * (k[1] - 1) + 1)) // s[1] + 1
        return oh, ow

    def input(self, name, c, h, w):
        x = synth.int8_uniform(self.g.seed, self._stream(0), (self.batch, c, h, w))
        op = self.g.add(Op("tpu.input", name, [], (self.batch, c, h, w)))
        op.data = x
        self.cal[name] = x[:1].astype(np.int64)
        self.layer += 1
        return name

    def conv(self, name, src, oc, k, stride=1, pad=None, groups=1, relu=False, sigma=32,
             bias_mag=4096, dil=1, pads=None, rshift_uniform=None):
        g = self.g
        n, ic, ih, iw = g.by_name[src].shape
        k = (k, k) if isinstance(k, int) else k
        s = (stride, stride) if isinstance(stride, int) else stride
        d = (dil, dil) if isinstance(dil, int) else dil
        if pads is None:
            p = (d[0] * (k[0] - 1)) // 2 if pad is None else pad
            pads = (p, p, p, p)
        oh, ow = self._out_hw(ih, iw, k, s, pads, d)
        icg = ic // groups
        seed = g.seed
        filt = synth.int8_normal(seed, self._stream(1), (oc, icg, k[0], k[1]), sigma)
        bias = synth.uniform_int(seed, self._stream(2), (oc,), -bias_mag, bias_mag)
        mult = synth.multipliers_q31(seed, self._stream(3), oc)
        # fp32-exactness guard of the reference's MKL-DNN accumulation
        worst = np.abs(filt.astype(np.int64)).reshape(oc, -1).sum(1) * 128 + np.abs(bias)
        assert worst.max() < (1 << 24), (name, int(worst.max()))
        acc = _conv_acc(self.cal[src], filt, s, pads, d, groups) + bias.reshape(1, oc, 1, 1)
        if rshift_uniform is not None:
            rsh = synth.uniform_int(seed, self._stream(4), (oc,), rshift_uniform[0],
                                    rshift_uniform[1])
        else:
            per_ch = np.sqrt(np.mean(acc.astype(np.float64) ** 2, axis=(0, 2, 3)))
            if oh * ow < 64:
                per_ch = np.full(oc, _rms(acc))
            per_ch = np.maximum(per_ch, 1.0)
            want = per_ch * (mult / float(1 << 31)) / TARGET_RMS
            rsh = np.clip(np.rint(np.log2(np.maximum(want, 1e-9))), self.rs_lo, self.rs_hi)
            rsh = rsh.astype(np.int64)
        y = _qdm(acc, mult.reshape(1, oc, 1, 1), rsh.reshape(1, oc, 1, 1))
        if relu:
            y = np.maximum(y, 0)
        attrs = dict(kernel_h=k[0], kernel_w=k[1], stride_h=s[0], stride_w=s[1], dilation_h=d[0],
                     dilation_w=d[1], padding_t=pads[0], padding_b=pads[1], padding_l=pads[2],
                     padding_r=pads[3], group=groups, is_dw=int(groups == ic and groups == oc and
                                                                 groups > 1),
                     with_bias=1, do_relu=int(relu), ins_h=0, ins_w=0, pad_value=0)
        wshape = (oc, icg, k[0], k[1]) if groups == 1 else (groups, oc // groups, icg, k[0], k[1])
        op = g.add(Op("tpu.conv_2d", name, [src], (n, oc, oh, ow), attrs,
                      dict(filter=filt.astype(np.float32).reshape(wshape),
                           bias=bias.astype(np.float32), rshift=rsh.astype(np.float32),
                           multiplier=mult.astype(np.float32)),
                      "RSHIFT_AND_M_I32"))
        op.macs = n * oc * oh * ow * icg * k[0] * k[1]
        g.macs += op.macs
        self.cal[name] = y
        _record(g, name, y)
        self.layer += 1
        return name

    def fc(self, name, src, n_out, relu=False, sigma=20, bias_mag=2048):
        g = self.g
        m, kdim = g.by_name[src].shape[0], int(np.prod(g.by_name[src].shape[1:]))
        seed = g.seed
        filt = synth.int8_normal(seed, self._stream(1), (n_out, kdim), sigma)
        bias = synth.uniform_int(seed, self._stream(2), (n_out,), -bias_mag, bias_mag)
        mult = int(synth.multipliers_q31(seed, self._stream(3), 1)[0])
        worst = np.abs(filt.astype(np.int64)).sum(1) * 128 + np.abs(bias)
        assert worst.max() < (1 << 24), (name, int(worst.max()))
        x = self.cal[src].reshape(1, kdim)
        acc = x @ filt.astype(np.int64).T + bias
        if relu:
            acc = np.maximum(acc, 0)
        want = max(_rms(acc), 1.0) * (mult / float(1 << 31)) / TARGET_RMS
        rsh = int(np.clip(round(math.log2(want)), self.rs_lo, self.rs_hi))
        y = _qdm(acc, np.int64(mult), np.int64(rsh))
        op = g.add(Op("tpu.fully_connected", name, [src], (m, n_out), dict(do_relu=int(relu)),
                      dict(filter=filt.astype(np.float32), bias=bias.astype(np.float32),
                           rshift=np.array([rsh], np.float32),
                           multiplier=np.array([mult], np.float32)),
                      "RSHIFT_AND_M_I32"))
        op.macs = m * n_out * kdim
        g.macs += op.macs
        self.cal[name] = y
        _record(g, name, y)
        self.layer += 1
        return name

    def add(self, name, srcs, relu):
        g = self.g
        seed = g.seed
        mult = synth.uniform_int(seed, self._stream(5), (len(srcs),), 40, 100)
        s = sum(self.cal[a] * int(m) for a, m in zip(srcs, mult))
        if relu:
            s = np.maximum(s, 0)
        rsh = int(np.clip(round(math.log2(max(_rms(s), 1.0) / TARGET_RMS)), 0, 14))
        y = np.clip(_half_up_shift(s, np.int64(rsh)), -128, 127)
        g.add(Op("tpu.eltwise_add", name, srcs, g.by_name[srcs[0]].shape, dict(do_relu=int(relu)),
                 dict(rshift=np.array([rsh], np.float32), multiplier=mult.astype(np.float32)),
                 "RSHIFT_AND_M_I8"))
        self.cal[name] = y
        _record(g, name, y)
        self.layer += 1
        return name

    def pool_max(self, name, src, k, stride, pads):
        g = self.g
        n, c, ih, iw = g.by_name[src].shape
        oh, ow = self._out_hw(ih, iw, (k, k), (stride, stride), pads)
        x = self.cal[src]
        xp = np.full((1, c, ih + pads[0] + pads[1], iw + pads[2] + pads[3]), -128, np.int64)
        xp[:, :, pads[0]:pads[0] + ih, pads[2]:pads[2] + iw] = x
        y = np.full((1, c, oh, ow), -128, np.int64)
        for i in range(k):
            for j in range(k):
                y = np.maximum(y, xp[:, :, i:i + stride * oh:stride, j:j + stride * ow:stride])
        g.add(Op("tpu.pool_max_2d", name, [src], (n, c, oh, ow),
                 dict(kernel_h=k, kernel_w=k, stride_h=stride, stride_w=stride, padding_t=pads[0],
                      padding_b=pads[1], padding_l=pads[2], padding_r=pads[3], do_relu=0,
                      count_include_pad=0, pad_value=0)))
        self.cal[name] = y
        self.layer += 1
        return name

    def global_avg(self, name, src):
        g = self.g
        n, c, ih, iw = g.by_name[src].shape
        s = self.cal[src].sum(axis=(2, 3), keepdims=True)
        rsh = 13
        mult = int(np.clip(round((1 << rsh) * TARGET_RMS / max(_rms(s), 1.0)), 1, 255))
        y = np.clip(_half_up_shift(s * mult, np.int64(rsh)), -128, 127)
        g.add(Op("tpu.pool_avg_2d", name, [src], (n, c, 1, 1),
                 dict(kernel_h=ih, kernel_w=iw, stride_h=1, stride_w=1, padding_t=0, padding_b=0,
                      padding_l=0, padding_r=0, do_relu=0, count_include_pad=1, pad_value=0),
                 dict(rshift=np.array([rsh], np.float32), multiplier=np.array([mult], np.float32)),
                 "RSHIFT_AND_M_I8"))
        self.cal[name] = y
        _record(g, name, y)
        self.layer += 1
        return name

    def reshape(self, name, src, shape):
        g = self.g
        g.add(Op("tpu.reshape", name, [src], shape))
        self.cal[name] = self.cal[src].reshape((1,) + tuple(shape[1:]))
        self.layer += 1
        return name

    def leaky(self, name, src):
        g = self.g
        pick = int(synth.uniform_int(g.seed, self._stream(6), (1,), 0, 2)[0])
        rp, mp = ((0, 1), (0, 1), (5, 31))[pick]
        rn, mn = ((7, 13), (8, 26), (7, 12))[pick]       # slope ~ 0.1
        x = self.cal[src]
        pos = np.clip(_half_up_shift(x * mp, np.int64(rp)), -128, 127)
        neg = np.clip(_half_up_shift(x * mn, np.int64(rn)), -128, 127)
        y = np.where(x > 0, pos, neg)
        g.add(Op("tpu.leaky_relu", name, [src], g.by_name[src].shape, dict(negative_slope=0.1),
                 dict(rshift_pos=np.array([rp], np.float32), multiplier_pos=np.array([mp], np.float32),
                      rshift_neg=np.array([rn], np.float32),
                      multiplier_neg=np.array([mn], np.float32)),
                 "RSHIFT_AND_M_I8"))
        self.cal[name] = y
        _record(g, name, y)
        self.layer += 1
        return name

    def clip(self, name, src, lo, hi):
        g = self.g
        g.add(Op("tpu.clip", name, [src], g.by_name[src].shape, dict(min=float(lo), max=float(hi)),
                 dict(rshift=np.array([0], np.float32), multiplier=np.array([1], np.float32)),
                 "RSHIFT_AND_M_I8"))
        self.cal[name] = np.clip(self.cal[src], lo, hi)
        _record(g, name, self.cal[name])
        self.layer += 1
        return name

    def upsample(self, name, src, scale):
        g = self.g
        n, c, h, w = g.by_name[src].shape
        g.add(Op("tpu.upsample", name, [src], (n, c, h * scale, w * scale),
                 dict(scale_h=scale, scale_w=scale)))
        self.cal[name] = np.repeat(np.repeat(self.cal[src], scale, 2), scale, 3)
        self.layer += 1
        return name

    def concat(self, name, srcs, axis=1):
        g = self.g
        shape = list(g.by_name[srcs[0]].shape)
        shape[axis] = sum(g.by_name[s].shape[axis] for s in srcs)
        g.add(Op("tpu.concat", name, srcs, shape, dict(axis=axis, do_relu=0)))
        self.cal[name] = np.concatenate([self.cal[s] for s in srcs], axis)
        self.layer += 1
        return name

    def finish(self, outputs):
        self.g.outputs = list(outputs)
        self.cal = {}
        return self.g


# ---------------------------------------------------------------------------
# the five configurations
# ---------------------------------------------------------------------------

BASE_SEED = 0x7C0DE000


def cfg1_single_conv(batch=1):
    """3x3 s1 p1 conv 64->64 at 56x56 with fused ReLU; rshift uniform on [8,20]."""
    b = Builder("cfg1_conv3x3", BASE_SEED + 1, batch, (8, 20))
    x = b.input("input", 64, 56, 56)
    y = b.conv("conv", x, 64, 3, relu=True, sigma=32, bias_mag=4096, rshift_uniform=(8, 20))
    return b.finish([y])


def cfg2_mobilenet_block(batch=8):
    """depthwise 3x3 on 256 channels, pointwise 256->256, each followed by requant + ReLU6
    realised as conv(do_relu) + an INT8 clip to [0, q6]."""
    b = Builder("cfg2_mobilenet_block", BASE_SEED + 2, batch, (4, 18))
    q6 = int(synth.uniform_int(b.g.seed, 0xFFFF, (1,), 64, 127)[0])
    x = b.input("input", 256, 56, 56)
    y = b.conv("dw", x, 256, 3, groups=256, relu=True, sigma=24, bias_mag=2048)
    y = b.clip("dw_relu6", y, 0, q6)
    y = b.conv("pw", y, 256, 1, relu=True, sigma=24, bias_mag=2048)
    y = b.clip("pw_relu6", y, 0, q6)
    return b.finish([y])


def cfg3_resnet50(batch=32, hw=224):
    """ResNet-50, Caffe variant (stride in the first 1x1 of a stage, ceil-mode pool1 ->
    pads 0,1,0,1): 53 convs, 16 residual adds, maxpool, global avgpool, FC 2048->1000."""
    b = Builder("cfg3_resnet50", BASE_SEED + 3, batch, (6, 18))
    x = b.input("input", 3, hw, hw)
    x = b.conv("conv1", x, 64, 7, stride=2, pad=3, relu=True)
    x = b.pool_max("pool1", x, 3, 2, (0, 1, 0, 1))
    stage_names = {0: "res2", 1: "res3", 2: "res4", 3: "res5"}
    for si, (blocks, mid) in enumerate(((3, 64), (4, 128), (6, 256), (3, 512))):
        for bi in range(blocks):
            p = "%s%s" % (stage_names[si], chr(ord("a") + bi))
            stride = 2 if (bi == 0 and si > 0) else 1
            if bi == 0:
                sc = b.conv(p + "_branch1", x, mid * 4, 1, stride=stride)
            else:
                sc = x
            y = b.conv(p + "_branch2a", x, mid, 1, stride=stride, relu=True)
            y = b.conv(p + "_branch2b", y, mid, 3, relu=True)
            y = b.conv(p + "_branch2c", y, mid * 4, 1)
            x = b.add(p, [sc, y], relu=True)
    x = b.global_avg("pool5", x)
    x = b.reshape("pool5_flat", x, (batch, b.g.by_name[x].shape[1]))
    x = b.fc("fc1000", x, 1000)
    return b.finish([x])


def cfg4_mobilenet_v2(batch=64, hw=224):
    """MobileNetV2: 17 inverted-residual blocks (expansion 6), 10 residual adds, 1x1 to
    1280, global avgpool, FC 1280->1000.  ReLU6 = conv do_relu + int8 saturation."""
    b = Builder("cfg4_mobilenet_v2", BASE_SEED + 4, batch, (4, 18))
    x = b.input("input", 3, hw, hw)
    x = b.conv("conv1", x, 32, 3, stride=2, relu=True)
    cin = 32
    idx = 0
    for t, c, n, s in ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1),
                       (6, 160, 3, 2), (6, 320, 1, 1)):
        for i in range(n):
            idx += 1
            stride = s if i == 0 else 1
            p = "block%d" % idx
            y = x
            if t != 1:
                y = b.conv(p + "_expand", y, cin * t, 1, relu=True)
            y = b.conv(p + "_dw", y, cin * t, 3, stride=stride, groups=cin * t, relu=True,
                       sigma=24)
            y = b.conv(p + "_project", y, c, 1)
            if stride == 1 and cin == c:
                y = b.add(p + "_add", [x, y], relu=False)
            x = y
            cin = c
    x = b.conv("conv_last", x, 1280, 1, relu=True)
    x = b.global_avg("pool", x)
    x = b.reshape("pool_flat", x, (batch, 1280))
    x = b.fc("fc", x, 1000)
    return b.finish([x])


def cfg5_yolo_v3(batch=8, hw=608):
    """YOLOv3: Darknet-53 backbone (52 convs, 23 residual adds) and three detection heads
    (19/38/76 grid at 608): 75 convs, 72 leaky-ReLUs, 2 upsamples, 2 concats."""
    b = Builder("cfg5_yolo_v3", BASE_SEED + 5, batch, (4, 18))
    counter = [0]

    def cbl(x, oc, k, stride=1, act=True):
        counter[0] += 1
        name = "conv%d" % counter[0]
        y = b.conv(name, x, oc, k, stride=stride, pad=k // 2)
        return b.leaky(name + "_leaky", y) if act else y

    x = b.input("input", 3, hw, hw)
    x = cbl(x, 32, 3)
    routes = {}
    for si, (oc, blocks) in enumerate(((64, 1), (128, 2), (256, 8), (512, 8), (1024, 4))):
        x = cbl(x, oc, 3, stride=2)
        for _ in range(blocks):
            y = cbl(x, oc // 2, 1)
            y = cbl(y, oc, 3)
            x = b.add("res%d" % counter[0], [x, y], relu=False)
        routes[si] = x
    outs = []

    def head(x, mid, tag):
        for _ in range(2):
            x = cbl(x, mid, 1)
            x = cbl(x, mid * 2, 3)
        x = cbl(x, mid, 1)
        y = cbl(x, mid * 2, 3)
        y = cbl(y, 255, 1, act=False)
        outs.append(y)
        return x

    x = head(x, 512, "l")
    x = cbl(x, 256, 1)
    x = b.upsample("upsample1", x, 2)
    x = b.concat("route1", [x, routes[3]])
    x = head(x, 256, "m")
    x = cbl(x, 128, 1)
    x = b.upsample("upsample2", x, 2)
    x = b.concat("route2", [x, routes[2]])
    head(x, 128, "s")
    return b.finish(outs)


CONFIGS = {
    "cfg1": cfg1_single_conv,
    "cfg2": cfg2_mobilenet_block,
    "cfg3": cfg3_resnet50,
    "cfg4": cfg4_mobilenet_v2,
    "cfg5": cfg5_yolo_v3,
}
