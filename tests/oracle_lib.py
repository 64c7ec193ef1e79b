"""ctypes view of oracle/libtpu_oracle.so (test infrastructure: the CPU checker).

Only tests, the smoke check and the CPU-baseline leg of the benchmark may use
this module.  Arrays are NCHW numpy int8; quantisation parameters are float32
arrays holding integers, the way the reference stores them.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_SO = os.path.join(ORACLE_DIR, "libtpu_oracle.so")


class ConvDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "n", "ic", "ih", "iw", "oc", "oh", "ow", "g", "kh", "kw", "sh", "sw",
        "pt", "pb", "pl", "pr", "dh", "dw", "ins_h", "ins_w", "do_relu", "with_bias")]


class PoolDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "n", "c", "ih", "iw", "oh", "ow", "kh", "kw", "sh", "sw", "pt", "pb", "pl", "pr")]


class BinaryDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "op", "n", "c", "h", "w", "n0", "c0", "h0", "w0", "n1", "c1", "h1", "w1", "do_relu")]


BIN_ADD, BIN_SUB, BIN_MAX, BIN_MIN, BIN_MUL = range(5)


def build():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR])


def _load():
    if not os.path.exists(_SO):
        build()
    lib = C.CDLL(_SO)
    i8p, f32p, i32p = C.POINTER(C.c_int8), C.POINTER(C.c_float), C.POINTER(C.c_int32)
    lib.orc_srdhm.restype = C.c_int32
    lib.orc_srdhm.argtypes = [C.c_int32, C.c_int32]
    lib.orc_rdbp.restype = C.c_int32
    lib.orc_rdbp.argtypes = [C.c_int32, C.c_int]
    lib.orc_saturate_int8.restype = C.c_int8
    lib.orc_saturate_int8.argtypes = [C.c_float]
    lib.orc_apply_rshift_sat8.restype = C.c_int8
    lib.orc_apply_rshift_sat8.argtypes = [C.c_float, C.c_uint32]
    lib.orc_apply_mult_rshift_sat8_f.restype = C.c_int8
    lib.orc_apply_mult_rshift_sat8_f.argtypes = [C.c_float, C.c_uint32, C.c_uint32, C.c_int]
    lib.orc_apply_mult_rshift_sat8_i.restype = C.c_int8
    lib.orc_apply_mult_rshift_sat8_i.argtypes = [C.c_int32, C.c_uint32, C.c_uint32, C.c_int]
    lib.orc_f2u32.restype = C.c_uint32
    lib.orc_f2u32.argtypes = [C.c_float]
    lib.orc_conv2d_acc.argtypes = [i8p, i8p, i32p, C.POINTER(ConvDesc)]
    lib.orc_conv2d_guard.restype = C.c_int64
    lib.orc_conv2d_guard.argtypes = [i8p, i8p, C.POINTER(ConvDesc)]
    lib.orc_conv2d_acc_f32.argtypes = [f32p, f32p, f32p, C.POINTER(ConvDesc)]
    lib.orc_requant_per_channel.argtypes = [i32p, i8p, f32p, C.c_int, C.c_int64, C.c_int64,
                                            C.c_int64, f32p, f32p]
    lib.orc_conv2d_i8.argtypes = [i8p, i8p, f32p, f32p, f32p, i8p, C.POINTER(ConvDesc)]
    lib.orc_deconv2d_acc.argtypes = [i8p, i8p, i32p, C.POINTER(ConvDesc)]
    lib.orc_deconv2d_i8.argtypes = [i8p, i8p, f32p, f32p, f32p, i8p, C.POINTER(ConvDesc)]
    lib.orc_quant_f32_to_i8.argtypes = [f32p, i8p, C.c_size_t, C.c_float]
    lib.orc_dequant_i8_to_f32.argtypes = [i8p, f32p, C.c_size_t, C.c_float]
    lib.orc_bf16.restype = C.c_float
    lib.orc_bf16.argtypes = [C.c_float, C.c_int]
    lib.orc_fc_i8.argtypes = [i8p, i8p, f32p, f32p, f32p, i8p] + [C.c_int] * 5
    lib.orc_fc_batched_i8.argtypes = [i8p, i8p, f32p, f32p, f32p, i8p] + [C.c_int] * 8
    lib.orc_fc_guard.restype = C.c_int64
    lib.orc_fc_guard.argtypes = [i8p, i8p, f32p] + [C.c_int] * 4
    lib.orc_eltwise_add_i8.argtypes = [C.POINTER(i8p), C.c_int, f32p, f32p, C.c_int, i8p,
                                       C.c_size_t]
    lib.orc_binary_i8.restype = C.c_int
    lib.orc_binary_i8.argtypes = [i8p, i8p, i8p, C.POINTER(BinaryDesc), f32p, C.c_float]
    i64p, ip = C.POINTER(C.c_int64), C.POINTER(C.c_int)
    lib.orc_pad_i8.argtypes = [i8p, i8p, i64p, ip, C.c_int]
    lib.orc_crop_i8.argtypes = [i8p, i8p, i64p, i64p, ip, ip]
    lib.orc_permute_i8.argtypes = [i8p, i8p, i64p, ip]
    lib.orc_reorg_i8.argtypes = [i8p, i8p, i64p, C.c_int]
    lib.orc_tile_i8.argtypes = [i8p, i8p, i64p, C.c_int, C.c_int]
    lib.orc_reverse_i8.argtypes = [i8p, i8p, i64p, C.c_int]
    lib.orc_dilate_i8.argtypes = [i8p, i8p, i64p, C.c_int, C.c_int, C.c_int]
    lib.orc_reflection_pad_i8.argtypes = [i8p, i8p, i64p, C.c_int, C.c_int]
    lib.orc_shuffle_channel_i8.argtypes = [i8p, i8p, i64p, C.c_int]
    lib.orc_depth_to_space_i8.argtypes = [i8p, i8p, i64p, C.c_int, C.c_int]
    lib.orc_swap_channel_i8.argtypes = [i8p, i8p, i64p, C.POINTER(C.c_int)]
    lib.orc_reduce_i8.argtypes = [C.c_int, i8p, i8p, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_float]
    lib.orc_lrn_i8.argtypes = [i8p, i8p] + [C.c_int] * 5 + [C.POINTER(C.c_float)] * 2 + [C.c_int] * 4
    lib.orc_zero_mask_i8.argtypes = [i8p, i8p, C.c_int64, C.c_int]
    lib.orc_mul_const_i8.argtypes = [i8p, i8p, C.c_int64, C.c_float, C.c_int]
    lib.orc_pool_max_i8.argtypes = [i8p, i8p, C.POINTER(PoolDesc)]
    lib.orc_pool_avg_i8.argtypes = [i8p, i8p, C.POINTER(PoolDesc), C.c_float, C.c_float]
    lib.orc_leaky_relu_i8.argtypes = [i8p, i8p, C.c_size_t] + [C.c_float] * 4
    lib.orc_prelu_i8.argtypes = [i8p, i8p, C.c_int, C.c_int, C.c_int, f32p] + [C.c_float] * 3
    lib.orc_lut_i8.argtypes = [i8p, i8p, C.c_size_t, f32p]
    lib.orc_relu_i8.argtypes = [i8p, i8p, C.c_size_t]
    lib.orc_clip_i8.argtypes = [i8p, i8p, C.c_size_t] + [C.c_float] * 4
    lib.orc_upsample_i8.argtypes = [i8p, i8p] + [C.c_int] * 6
    lib.orc_concat_i8.argtypes = [C.POINTER(i8p), C.c_int, C.POINTER(C.c_int64), C.c_int, C.c_int,
                                  f32p, f32p, C.c_int, i8p]
    return lib


lib = _load()


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t)) if a is not None else None


def _i8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.int8, a.dtype
    return a


def _f32(a):
    if a is None:
        return None
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).reshape(-1))


def conv_out_hw(ih, iw, kh, kw, sh, sw, pt, pb, pl, pr, dh=1, dw=1, ins_h=0, ins_w=0):
    ihd = (ih - 1) * (ins_h + 1) + 1
    iwd = (iw - 1) * (ins_w + 1) + 1
    oh = (ihd + pt + pb - (dh * (kh - 1) + 1)) // sh + 1
    ow = (iwd + pl + pr - (dw * (kw - 1) + 1)) // sw + 1
    return oh, ow


def make_conv_desc(x_shape, w_shape, g=1, stride=(1, 1), pads=(0, 0, 0, 0), dil=(1, 1),
                   ins=(0, 0), do_relu=False, with_bias=True, out_hw=None):
    n, ic, ih, iw = x_shape
    oc = w_shape[0]
    kh, kw = w_shape[-2], w_shape[-1]
    pt, pb, pl, pr = pads
    oh, ow = out_hw or conv_out_hw(ih, iw, kh, kw, stride[0], stride[1], pt, pb, pl, pr,
                                   dil[0], dil[1], ins[0], ins[1])
    return ConvDesc(n, ic, ih, iw, oc, oh, ow, g, kh, kw, stride[0], stride[1], pt, pb, pl, pr,
                    dil[0], dil[1], ins[0], ins[1], int(do_relu), int(with_bias))


def conv2d_acc(x, w, d):
    x, w = _i8(x), _i8(w)
    acc = np.empty((d.n, d.oc, d.oh, d.ow), np.int32)
    lib.orc_conv2d_acc(_p(x, C.c_int8), _p(w, C.c_int8), _p(acc, C.c_int32), C.byref(d))
    return acc


def conv2d_guard(x, w, d):
    x, w = _i8(x), _i8(w)
    return int(lib.orc_conv2d_guard(_p(x, C.c_int8), _p(w, C.c_int8), C.byref(d)))


def conv2d_acc_f32(x, w, d):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    acc = np.empty((d.n, d.oc, d.oh, d.ow), np.float32)
    lib.orc_conv2d_acc_f32(_p(x, C.c_float), _p(w, C.c_float), _p(acc, C.c_float), C.byref(d))
    return acc


def requant_per_channel(acc, bias, rshift, multiplier, do_relu):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    n, oc = acc.shape[0], acc.shape[1]
    isz = int(np.prod(acc.shape[2:])) if acc.ndim > 2 else 1
    y = np.empty(acc.shape, np.int8)
    b, r, m = _f32(bias), _f32(rshift), _f32(multiplier)
    lib.orc_requant_per_channel(_p(acc, C.c_int32), _p(y, C.c_int8), _p(b, C.c_float),
                                int(do_relu), n, oc, isz, _p(r, C.c_float), _p(m, C.c_float))
    return y


def conv2d_i8(x, w, bias, rshift, multiplier, d):
    x, w = _i8(x), _i8(w)
    y = np.empty((d.n, d.oc, d.oh, d.ow), np.int8)
    b, r, m = _f32(bias), _f32(rshift), _f32(multiplier)
    lib.orc_conv2d_i8(_p(x, C.c_int8), _p(w, C.c_int8), _p(b, C.c_float), _p(r, C.c_float),
                      _p(m, C.c_float), _p(y, C.c_int8), C.byref(d))
    return y


def fc_i8(x, w, bias, rshift, multiplier, batch, m, k, n, do_relu):
    x, w = _i8(x), _i8(w)
    y = np.empty((batch, m, n), np.int8)
    b, r, mu = _f32(bias), _f32(rshift), _f32(multiplier)
    lib.orc_fc_i8(_p(x, C.c_int8), _p(w, C.c_int8), _p(b, C.c_float), _p(r, C.c_float),
                  _p(mu, C.c_float), _p(y, C.c_int8), batch, m, k, n, int(do_relu))
    return y


def fc_batched_i8(x, w, bias, rshift, multiplier, batch_high, batch_low, m, k, n, ltrans, otrans, do_relu):
    """x in the input's logical order; returns the result flat in ITS logical order"""
    x, w = _i8(x), _i8(w)
    batch = batch_high * batch_low
    assert x.size == batch * m * k and w.size == batch * n * k
    y = np.empty(batch * m * n, np.int8)
    b, r, mu = _f32(bias), _f32(rshift), _f32(multiplier)
    lib.orc_fc_batched_i8(_p(x, C.c_int8), _p(w, C.c_int8), _p(b, C.c_float), _p(r, C.c_float),
                          _p(mu, C.c_float), _p(y, C.c_int8), batch_high, batch_low, m, k, n,
                          int(ltrans), int(otrans), int(do_relu))
    return y


def fc_guard(x, w, bias, batch, m, k, n):
    x, w = _i8(x), _i8(w)
    b = _f32(bias)
    return int(lib.orc_fc_guard(_p(x, C.c_int8), _p(w, C.c_int8), _p(b, C.c_float), batch, m, k, n))


def _ptr_array(arrs):
    arr_t = C.POINTER(C.c_int8) * len(arrs)
    return arr_t(*[_p(a, C.c_int8) for a in arrs])


def eltwise_add_i8(xs, multiplier, rshift, do_relu):
    xs = [_i8(a) for a in xs]
    y = np.empty(xs[0].shape, np.int8)
    m, r = _f32(multiplier), _f32(rshift)
    lib.orc_eltwise_add_i8(_ptr_array(xs), len(xs), _p(m, C.c_float), _p(r, C.c_float),
                           int(do_relu), _p(y, C.c_int8), xs[0].size)
    return y


def make_deconv_desc(x_shape, w_shape, g, stride, pads, dil, out_hw, do_relu=False, with_bias=True):
    """w_shape = (oc, ic // g, kh, kw); out_hw is the op's result size"""
    n, ic, ih, iw = x_shape
    return ConvDesc(n, ic, ih, iw, w_shape[0], out_hw[0], out_hw[1], g, w_shape[2], w_shape[3],
                    stride[0], stride[1], pads[0], pads[1], pads[2], pads[3], dil[0], dil[1], 0, 0,
                    int(do_relu), int(with_bias))


def deconv2d_acc(x, w, d):
    x, w = _i8(x), _i8(w)
    acc = np.empty((d.n, d.oc, d.oh, d.ow), np.int32)
    lib.orc_deconv2d_acc(_p(x, C.c_int8), _p(w, C.c_int8), _p(acc, C.c_int32), C.byref(d))
    return acc


def deconv2d_i8(x, w, bias, rshift, multiplier, d):
    x, w = _i8(x), _i8(w)
    y = np.empty((d.n, d.oc, d.oh, d.ow), np.int8)
    b = _f32(bias) if bias is not None else None
    lib.orc_deconv2d_i8(_p(x, C.c_int8), _p(w, C.c_int8), _p(b, C.c_float) if b is not None else None,
                        _p(_f32(rshift), C.c_float), _p(_f32(multiplier), C.c_float),
                        _p(y, C.c_int8), C.byref(d))
    return y


def quant_f32_to_i8(x, scale):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, np.int8)
    lib.orc_quant_f32_to_i8(_p(x, C.c_float), _p(y, C.c_int8), x.size, float(scale))
    return y


def dequant_i8_to_f32(x, scale):
    x = _i8(x)
    y = np.empty(x.shape, np.float32)
    lib.orc_dequant_i8_to_f32(_p(x, C.c_int8), _p(y, C.c_float), x.size, float(scale))
    return y


def _shape64(shape):
    return (C.c_int64 * 4)(*shape)


def _ints(v):
    return (C.c_int * len(v))(*[int(a) for a in v])


def move_i8(kind, x, params, out_shape=None):
    """the data movement ops by name: pad_const, pad_edge, crop, permute, reorg, tile, reverse,
    shuffle_channel, depth_to_space (params as in the C ABI's tpuhip_move_desc.p)"""
    x = _i8(x)
    s, p = x.shape, [int(v) for v in params]
    if kind in ("pad_const", "pad_edge"):
        out = tuple(s[k] + p[k] + p[4 + k] for k in range(4))
    elif kind == "crop":
        out = tuple(out_shape)
    elif kind == "permute":
        out = tuple(s[p[k]] for k in range(4))
    elif kind == "reorg":
        out = (s[0], s[1] * p[0] * p[0], s[2] // p[0], s[3] // p[0])
    elif kind == "tile":
        out = tuple(s[k] * (p[1] if k == p[0] else 1) for k in range(4))
    elif kind in ("reverse", "shuffle_channel", "swap_channel"):
        out = s
    elif kind == "dilate":      # p = ins_w, ins_h, fill_constant
        out = (s[0], s[1], (s[2] - 1) * (p[1] + 1) + 1, (s[3] - 1) * (p[0] + 1) + 1)
    elif kind == "reflection_pad":
        out = (s[0], s[1], s[2], s[3] + p[0] + p[1])
    else:
        out = (s[0], s[1] // (p[0] * p[0]), s[2] * p[0], s[3] * p[0])
    y = np.empty(out, np.int8)
    xp, yp = _p(x, C.c_int8), _p(y, C.c_int8)
    if kind in ("pad_const", "pad_edge"):
        lib.orc_pad_i8(xp, yp, _shape64(s), _ints(p[:8]), int(kind == "pad_edge"))
    elif kind == "crop":
        lib.orc_crop_i8(xp, yp, _shape64(s), _shape64(out), _ints(p[:4]), _ints(p[4:8]))
    elif kind == "permute":
        lib.orc_permute_i8(xp, yp, _shape64(s), _ints(p[:4]))
    elif kind == "reorg":
        lib.orc_reorg_i8(xp, yp, _shape64(s), p[0])
    elif kind == "tile":
        lib.orc_tile_i8(xp, yp, _shape64(s), p[0], p[1])
    elif kind == "reverse":
        lib.orc_reverse_i8(xp, yp, _shape64(s), p[0])
    elif kind == "shuffle_channel":
        lib.orc_shuffle_channel_i8(xp, yp, _shape64(s), p[0])
    elif kind == "swap_channel":
        lib.orc_swap_channel_i8(xp, yp, _shape64(s), _ints(p[:s[1]]))
    elif kind == "dilate":
        lib.orc_dilate_i8(xp, yp, _shape64(s), p[1], p[0], p[2])
    elif kind == "reflection_pad":
        lib.orc_reflection_pad_i8(xp, yp, _shape64(s), p[0], p[1])
    else:
        lib.orc_depth_to_space_i8(xp, yp, _shape64(s), p[0], p[1])
    return y


MOVE_KINDS = ["pad_const", "pad_edge", "crop", "permute", "reorg", "tile", "reverse",
              "shuffle_channel", "depth_to_space", "swap_channel", "dilate", "reflection_pad"]


def lrn_i8(x, local_size, sqr_lut, power_lut, sum_rshift, lrn_rshift, quant0, quant1):
    x = _i8(x)
    y = np.empty(x.shape, np.int8)
    sq, pw = _f32(sqr_lut), _f32(power_lut)
    n, c, h, w = x.shape
    lib.orc_lrn_i8(_p(x, C.c_int8), _p(y, C.c_int8), n, c, h, w, int(local_size), _p(sq, C.c_float),
                   _p(pw, C.c_float), int(sum_rshift), int(lrn_rshift), int(quant0), int(quant1))
    return y


REDUCE_KINDS = {"mean": 0, "sum": 1, "max": 2, "min": 3}


def reduce_i8(kind, x, axes, out_shape, rshift=0, multiplier=1):
    """reduce over consecutive axes of an NCHW tensor; out_shape as the op declares it"""
    x = _i8(x)
    axes = [int(a) for a in axes]
    assert axes == list(range(axes[0], axes[-1] + 1))
    outer = int(np.prod(x.shape[:axes[0]], dtype=np.int64))
    axis = int(np.prod(x.shape[axes[0]:axes[-1] + 1], dtype=np.int64))
    inner = int(np.prod(x.shape[axes[-1] + 1:], dtype=np.int64))
    y = np.empty(tuple(out_shape), np.int8)
    assert y.size == outer * inner
    lib.orc_reduce_i8(REDUCE_KINDS[kind], _p(x, C.c_int8), _p(y, C.c_int8), outer, axis, inner,
                      float(rshift), float(multiplier))
    return y


def zero_mask_i8(x, positive):
    x = _i8(x)
    y = np.empty(x.shape, np.int8)
    lib.orc_zero_mask_i8(_p(x, C.c_int8), _p(y, C.c_int8), x.size, int(bool(positive)))
    return y


def mul_const_i8(x, const_val, do_relu=False):
    x = _i8(x)
    y = np.empty(x.shape, np.int8)
    lib.orc_mul_const_i8(_p(x, C.c_int8), _p(y, C.c_int8), x.size, float(const_val), int(bool(do_relu)))
    return y


def prelu_i8(x, slope, rshift_pos, multiplier_pos, rshift_neg):
    x = _i8(x)
    n, c = x.shape[0], x.shape[1]
    y = np.empty(x.shape, np.int8)
    sl = _f32(slope)
    lib.orc_prelu_i8(_p(x, C.c_int8), _p(y, C.c_int8), n, c, x.size // (n * c), _p(sl, C.c_float),
                     float(rshift_pos), float(multiplier_pos), float(rshift_neg))
    return y


def scale_lut_u8(x, table):
    """x: uint8 NCHW; table: c * 256 float-stored int8 entries"""
    x = np.ascontiguousarray(x, np.uint8)
    n, c = x.shape[0], x.shape[1]
    t = _f32(table)
    assert t.size >= c * 256
    y = np.empty(x.shape, np.int8)
    lib.orc_scale_lut_u8(_p(x, C.c_uint8), _p(y, C.c_int8), n, c, x.size // (n * c), _p(t, C.c_float))
    return y


def binary_i8(op, x0, x1, multiplier, rshift, do_relu=False):
    """two-input elementwise op with broadcasting; x0, x1 4-d NCHW int8 (dims 1 broadcast)"""
    x0, x1 = _i8(x0), _i8(x1)
    out = tuple(max(a, b) for a, b in zip(x0.shape, x1.shape))
    d = BinaryDesc(op, *out, *x0.shape, *x1.shape, int(do_relu))
    y = np.empty(out, np.int8)
    m = _f32(multiplier)
    rc = lib.orc_binary_i8(_p(x0, C.c_int8), _p(x1, C.c_int8), _p(y, C.c_int8), C.byref(d),
                           _p(m, C.c_float), float(rshift))
    if rc != 0:
        raise ValueError("orc_binary_i8: no int8 meaning (mul with rshift 0 and multiplier 0)")
    return y


def make_pool_desc(x_shape, k, s, pads, out_hw=None):
    n, c, ih, iw = x_shape
    pt, pb, pl, pr = pads
    oh, ow = out_hw or ((ih + pt + pb - k[0]) // s[0] + 1, (iw + pl + pr - k[1]) // s[1] + 1)
    return PoolDesc(n, c, ih, iw, oh, ow, k[0], k[1], s[0], s[1], pt, pb, pl, pr)


def pool_max_i8(x, d):
    x = _i8(x)
    y = np.empty((d.n, d.c, d.oh, d.ow), np.int8)
    lib.orc_pool_max_i8(_p(x, C.c_int8), _p(y, C.c_int8), C.byref(d))
    return y


def pool_avg_i8(x, d, rshift, multiplier):
    x = _i8(x)
    y = np.empty((d.n, d.c, d.oh, d.ow), np.int8)
    lib.orc_pool_avg_i8(_p(x, C.c_int8), _p(y, C.c_int8), C.byref(d), float(rshift),
                        float(multiplier))
    return y


def leaky_relu_i8(x, rshift_pos, multiplier_pos, rshift_neg, multiplier_neg):
    x = _i8(x)
    y = np.empty(x.shape, np.int8)
    lib.orc_leaky_relu_i8(_p(x, C.c_int8), _p(y, C.c_int8), x.size, float(rshift_pos),
                          float(multiplier_pos), float(rshift_neg), float(multiplier_neg))
    return y


def lut_i8(x, table256):
    x = _i8(x)
    t = _f32(table256)
    assert t.size >= 256
    y = np.empty(x.shape, np.int8)
    lib.orc_lut_i8(_p(x, C.c_int8), _p(y, C.c_int8), x.size, _p(t, C.c_float))
    return y


def relu_i8(x):
    x = _i8(x)
    y = np.empty(x.shape, np.int8)
    lib.orc_relu_i8(_p(x, C.c_int8), _p(y, C.c_int8), x.size)
    return y


def clip_i8(x, lo, hi, rshift, multiplier):
    x = _i8(x)
    y = np.empty(x.shape, np.int8)
    lib.orc_clip_i8(_p(x, C.c_int8), _p(y, C.c_int8), x.size, float(lo), float(hi),
                    float(rshift), float(multiplier))
    return y


def upsample_i8(x, scale_h, scale_w):
    x = _i8(x)
    n, c, ih, iw = x.shape
    y = np.empty((n, c, ih * scale_h, iw * scale_w), np.int8)
    lib.orc_upsample_i8(_p(x, C.c_int8), _p(y, C.c_int8), n, c, ih, iw, scale_h, scale_w)
    return y


def concat_i8(xs, axis, rshift=None, multiplier=None, do_relu=False):
    xs = [_i8(a) for a in xs]
    ndim = xs[0].ndim
    shapes = np.ascontiguousarray(np.array([a.shape for a in xs], dtype=np.int64))
    out_shape = list(xs[0].shape)
    out_shape[axis] = int(sum(a.shape[axis] for a in xs))
    y = np.empty(out_shape, np.int8)
    r, m = _f32(rshift), _f32(multiplier)
    lib.orc_concat_i8(_ptr_array(xs), len(xs), _p(shapes, C.c_int64), ndim, axis,
                      _p(r, C.c_float), _p(m, C.c_float), int(do_relu), _p(y, C.c_int8))
    return y
