"""Helpers for the GPU parity tests: drive the tpuhip C ABI from numpy NCHW
arrays so results can be compared with the oracle's."""
import numpy as np

from tpu_compiler_amd import capi


def f2i32(values):
    """float-stored parameter -> the int32 the reference's epilogue ends up using:
    (int32_t)(uint32_t)float, the float -> uint32 step as x86-64 gcc compiles it."""
    v = np.asarray(values, dtype=np.float32).astype(np.int64)
    return (v & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


def conv_desc(x_shape, w_shape, g=1, stride=(1, 1), pads=(0, 0, 0, 0), dil=(1, 1), ins=(0, 0),
              do_relu=False, with_bias=True, out_hw=None, algo=0, relu_first=0, x_cs=None,
              y_cs=None):
    n, ic, ih, iw = x_shape
    oc, kh, kw = w_shape[0], w_shape[-2], w_shape[-1]
    pt, pb, pl, pr = pads
    ihd, iwd = (ih - 1) * (ins[0] + 1) + 1, (iw - 1) * (ins[1] + 1) + 1
    if out_hw is None:
        oh = (ihd + pt + pb - (dil[0] * (kh - 1) + 1)) // stride[0] + 1
        ow = (iwd + pl + pr - (dil[1] * (kw - 1) + 1)) // stride[1] + 1
    else:
        oh, ow = out_hw
    return capi.ConvDesc(n, ic, ih, iw, oc, oh, ow, g, kh, kw, stride[0], stride[1], pt, pb, pl,
                         pr, dil[0], dil[1], ins[0], ins[1], int(do_relu), int(with_bias),
                         x_cs or capi.channel_stride(ic), y_cs or capi.channel_stride(oc),
                         relu_first, algo)


def run_conv(ctx, x, w, bias_f, rshift_f, mult_f, algo=0, check_pad=True, **kw):
    d = conv_desc(x.shape, w.shape, algo=algo, **kw)
    xt = ctx.from_nchw(x)
    yt = ctx.tensor((d.n, d.oc, d.oh, d.ow))
    ctx._ck(ctx.lib.tpuhip_memset(ctx.h, yt.ptr, 0x55, yt.nbytes))  # poison: pads must be rewritten
    bias = None if bias_f is None else f2i32(bias_f)
    wh = ctx.conv_prepack(d, w, bias, f2i32(mult_f), f2i32(rshift_f))
    name = ctx.conv_algo_name(wh)
    ctx.conv(wh, xt, yt)
    y = ctx.to_nchw(yt)
    if check_pad and yt.cs != d.oc:
        raw = ctx.raw(yt)
        assert not raw[..., d.oc:].any(), "pad channels must be zero"
    ctx.conv_weights_destroy(wh)
    xt.free()
    yt.free()
    return y, name


def pool_desc(x_shape, k, s, pads, out_hw=None):
    n, c, ih, iw = x_shape
    pt, pb, pl, pr = pads
    oh, ow = out_hw or ((ih + pt + pb - k[0]) // s[0] + 1, (iw + pl + pr - k[1]) // s[1] + 1)
    cs = capi.channel_stride(c)
    return capi.PoolDesc(n, c, ih, iw, oh, ow, k[0], k[1], s[0], s[1], pt, pb, pl, pr, cs, cs)
