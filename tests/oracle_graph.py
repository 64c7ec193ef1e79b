"""Runs a graphs.Graph through the CPU oracle (test infrastructure): NCHW int8
tensors, every op's result kept, so the GPU run can be compared layer by layer."""
import numpy as np

import oracle_lib as O


def _conv(op, x):
    a = op.attrs
    w = op.weights["filter"].astype(np.int8)
    g = int(a["group"])
    oc = op.shape[1]
    w = w.reshape(oc, -1, int(a["kernel_h"]), int(a["kernel_w"]))
    d = O.make_conv_desc(
        x.shape, w.shape, g, (int(a["stride_h"]), int(a["stride_w"])),
        (int(a["padding_t"]), int(a["padding_b"]), int(a["padding_l"]), int(a["padding_r"])),
        (int(a["dilation_h"]), int(a["dilation_w"])), (int(a.get("ins_h", 0)), int(a.get("ins_w", 0))),
        bool(a["do_relu"]), bool(a["with_bias"]), (op.shape[2], op.shape[3]))
    return O.conv2d_i8(x, w, op.weights.get("bias"), op.weights["rshift"],
                       op.weights["multiplier"], d), d, w


_BINARY = {"tpu.eltwise_max": O.BIN_MAX, "tpu.eltwise_min": O.BIN_MIN, "tpu.eltwise_mul": O.BIN_MUL,
           "tpu.broadcast_add": O.BIN_ADD, "tpu.broadcast_sub": O.BIN_SUB,
           "tpu.broadcast_mul": O.BIN_MUL}


_MOVES = {"tpu.pad": ("pad_const", ["pads*"]), "tpu.crop": ("crop", ["crop_offset*", "steps*"]),
          "tpu.swap_channel": ("swap_channel", ["channel_order*"]),
          "tpu.dilate": ("dilate", ["ins0", "ins1", "fill_constant"]),
          "tpu.reflection_pad": ("reflection_pad", ["pads0", "pads1"]),
          "tpu.permute": ("permute", ["order*"]), "tpu.reorg": ("reorg", ["stride"]),
          "tpu.tile": ("tile", ["axis", "tiles"]), "tpu.reverse": ("reverse", ["axis"]),
          "tpu.shuffle_channel": ("shuffle_channel", ["group"]),
          "tpu.pixelshuffle": ("depth_to_space", ["upscale_factor", "mode_dcr"])}


def fc_params(a_s, b_s, o_s, ltrans, otrans):
    """parseFullyConnectedParam (lib/Dialect/TPU/IR/TPUOperationSupport.cpp:568-605)"""
    o_dim = len(o_s)
    k, n = int(b_s[-1]), int(b_s[-2])
    bl = bh = 1
    if ltrans:
        bl, m, bh = int(a_s[o_dim - 2]), int(a_s[o_dim - 3]), int(np.prod(a_s[:o_dim - 3], dtype=np.int64))
    elif otrans:
        bl, m, bh = int(o_s[o_dim - 2]), int(o_s[o_dim - 3]), int(np.prod(o_s[:o_dim - 3], dtype=np.int64))
    else:
        bl = int(np.prod(b_s[:-2], dtype=np.int64))
        m = int(a_s[o_dim - 2]) if bl > 1 else int(np.prod(a_s[:o_dim - 1], dtype=np.int64))
    return bh, bl, m, k, n


def run(graph, input_data=None, upto=None, keep=None, batch_slice=None, guards=None):
    """Returns {name: int8 NCHW array}.  batch_slice selects images (ops are
    independent across the batch, which is also how the reference runs a batch:
    one N=1 pass per slot).  guards: dict filled with the fp32-exactness guard of
    every conv / fc when given."""
    vals = {}
    for op in graph.ops:
        ins = [vals[n] for n in op.inputs]
        t = op.type
        if t == "tpu.input":
            y = op.data if input_data is None else input_data
            if batch_slice is not None:
                y = np.ascontiguousarray(y[batch_slice])
        elif t == "tpu.conv_2d":
            y, d, w = _conv(op, ins[0])
            if guards is not None:
                guards[op.name] = O.conv2d_guard(ins[0], w, d) + int(
                    np.abs(op.weights["bias"]).max())
        elif t == "tpu.deconv_2d":
            a = op.attrs
            w = op.weights["filter"].astype(np.int8)
            g_ = int(a.get("group", 1))
            w = w.reshape(op.shape[1], ins[0].shape[1] // g_, int(a["kernel_h"]), int(a["kernel_w"]))
            d = O.make_deconv_desc(ins[0].shape, w.shape, g_, (int(a["stride_h"]), int(a["stride_w"])),
                                   (int(a["padding_t"]), int(a["padding_b"]), int(a["padding_l"]),
                                    int(a["padding_r"])),
                                   (int(a.get("dilation_h", 1)), int(a.get("dilation_w", 1))),
                                   (op.shape[2], op.shape[3]), bool(a.get("do_relu", 0)),
                                   bool(a.get("with_bias", 1)))
            y = O.deconv2d_i8(ins[0], w, op.weights.get("bias"), op.weights["rshift"],
                              op.weights["multiplier"], d)
        elif t == "tpu.fully_connected":
            w = op.weights["filter"].astype(np.int8)
            lt, ot = int(op.attrs.get("input_transpose", 0)), int(op.attrs.get("output_transpose", 0))
            if w.ndim == 2 and len(op.shape) == 2 and not lt and not ot:
                x = ins[0].reshape(ins[0].shape[0], -1)
                y = O.fc_i8(x, w, op.weights.get("bias"), op.weights["rshift"],
                            op.weights["multiplier"], 1, x.shape[0], x.shape[1], w.shape[0],
                            bool(op.attrs.get("do_relu", 0)))[0]
                if guards is not None:
                    guards[op.name] = O.fc_guard(x, w, op.weights.get("bias"), 1, x.shape[0],
                                                 x.shape[1], w.shape[0])
            else:
                bh, bl, m, k, n = fc_params(ins[0].shape, w.shape, op.shape, lt, ot)
                y = O.fc_batched_i8(ins[0], w, op.weights.get("bias"), op.weights["rshift"],
                                    op.weights["multiplier"], bh, bl, m, k, n, lt, ot,
                                    bool(op.attrs.get("do_relu", 0))).reshape(op.shape)
                if guards is not None:
                    xb = ins[0].reshape(bh, m, bl, k).transpose(0, 2, 1, 3) if lt else ins[0]
                    guards[op.name] = O.fc_guard(np.ascontiguousarray(xb), w, op.weights.get("bias"),
                                                 bh * bl, m, k, n)
        elif t == "tpu.eltwise_add":
            y = O.eltwise_add_i8(ins, op.weights["multiplier"], op.weights["rshift"],
                                 bool(op.attrs.get("do_relu", 0)))
        elif t in _BINARY:
            def nchw(a):
                return a.reshape(a.shape + (1,) * (4 - a.ndim))
            y = O.binary_i8(_BINARY[t], nchw(ins[0]), nchw(ins[1]), op.weights["multiplier"],
                            op.weights["rshift"][0], bool(op.attrs.get("do_relu", 0)))
            y = y.reshape(op.shape)
        elif t in ("tpu.pool_max_2d", "tpu.pool_avg_2d"):
            a = op.attrs
            d = O.make_pool_desc(ins[0].shape, (int(a["kernel_h"]), int(a["kernel_w"])),
                                 (int(a["stride_h"]), int(a["stride_w"])),
                                 (int(a["padding_t"]), int(a["padding_b"]), int(a["padding_l"]),
                                  int(a["padding_r"])), (op.shape[2], op.shape[3]))
            if t == "tpu.pool_max_2d":
                y = O.pool_max_i8(ins[0], d)
            else:
                y = O.pool_avg_i8(ins[0], d, op.weights["rshift"][0], op.weights["multiplier"][0])
        elif t == "tpu.leaky_relu":
            w = op.weights
            y = O.leaky_relu_i8(ins[0], w["rshift_pos"][0], w["multiplier_pos"][0],
                                w["rshift_neg"][0], w["multiplier_neg"][0])
        elif t == "tpu.permute" and ins[0].ndim != 4:
            # core/permute.cpp:8-44 behind parsePermuteParam's folding to 4-d
            # (TPUOperationSupport.cpp:690-737): result dimension d is input dimension order[d]
            order = [int(op.attrs["order%d" % d]) for d in range(ins[0].ndim)]
            y = np.ascontiguousarray(np.transpose(ins[0], order))
        elif t in _MOVES:
            a = op.attrs
            kind, keys = _MOVES[t]
            if t == "tpu.pad" and a.get("mode_edge", 0):
                kind = "pad_edge"
            params = []
            for k in keys:
                if k.endswith("*"):
                    base, dflt = k[:-1], (1 if k.startswith("steps") else 0)
                    cnt = 8 if k.startswith("pads") else ins[0].shape[1] if k.startswith("channel_order") else 4
                    params += [int(a.get(base + str(i), dflt)) for i in range(cnt)]
                else:
                    params.append(int(a.get(k, 0)))
            y = O.move_i8(kind, ins[0], params, op.shape)
        elif t == "tpu.quant":
            if op.quant == "INT8":
                y = O.quant_f32_to_i8(ins[0], op.attrs["scale"])
            else:
                y = O.dequant_i8_to_f32(ins[0], op.attrs["scale"])
        elif t == "tpu.scale_lut":
            y = O.scale_lut_u8(ins[0], op.weights["table"])
        elif t == "tpu.prelu":
            w = op.weights
            y = O.prelu_i8(ins[0], w["slope"], w["rshift_pos"][0], w["multiplier_pos"][0],
                           w["rshift_neg"][0])
        elif t == "tpu.clip":
            y = O.clip_i8(ins[0], op.attrs["min"], op.attrs["max"], op.weights["rshift"][0],
                          op.weights["multiplier"][0])
        elif t == "tpu.lut" or (op.param_type == "LUT_INT8" and "table" in op.weights):
            # sigmoid, tanh, exp, ... in INT8 are all one 256-entry table lookup
            y = O.lut_i8(ins[0], op.weights["table"])
        elif t == "tpu.relu":
            y = O.relu_i8(ins[0])
        elif t in ("tpu.reduce_mean", "tpu.reduce_sum", "tpu.reduce_max", "tpu.reduce_min"):
            axes = [int(op.attrs["axes%d" % k]) for k in range(4) if "axes%d" % k in op.attrs]
            full = (ins[0].shape[0],) + tuple(op.shape[1:])
            y = O.reduce_i8(t[len("tpu.reduce_"):], ins[0], axes, full,
                            op.weights["rshift"][0] if "rshift" in op.weights else 0,
                            op.weights["multiplier"][0] if "multiplier" in op.weights else 1)
        elif t == "tpu.lrn":
            a = op.attrs
            y = O.lrn_i8(ins[0], a["local_size"], op.weights["sqr_lut"], op.weights["power_lut"], a["sum_rshift"],
                         a["lrn_rshift"], a["quant_data0"], a["quant_data1"])
        elif t == "tpu.zero_mask":
            y = O.zero_mask_i8(ins[0], op.attrs.get("positive", 0))
        elif t == "tpu.mul_const":
            y = O.mul_const_i8(ins[0], op.attrs["const_val"], op.attrs.get("do_relu", 0))
        elif t == "tpu.upsample":
            y = O.upsample_i8(ins[0], int(op.attrs["scale_h"]), int(op.attrs["scale_w"]))
        elif t == "tpu.concat":
            y = O.concat_i8(ins, int(op.attrs["axis"]), op.weights.get("rshift"),
                            op.weights.get("multiplier"), bool(op.attrs.get("do_relu", 0)))
        elif t == "tpu.reshape":
            full = ins[0].size == int(np.prod(op.shape))
            y = ins[0].reshape(tuple(op.shape) if full else (ins[0].shape[0],) + tuple(op.shape[1:]))
        else:
            raise NotImplementedError(t)
        vals[op.name] = y
        if upto is not None and op.name == upto:
            break
    if keep is not None:
        return {k: vals[k] for k in keep}
    return vals
