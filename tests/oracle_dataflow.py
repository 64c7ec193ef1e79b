"""The reference interpreter's DATA FLOW restated on the CPU (test infrastructure, the timed
CPU baseline of the benchmark): every tensor is float32 NCHW holding integers, convolutions,
inner products and pools run in fp32 through oneDNN (PyTorch's CPU ops -- the successor of the
MKL-DNN 1.0.2 the reference links), and the float / integer epilogues follow.

The graph is run the way the reference runs a batch: as an N=1 graph, once per image
(lib/Dialect/TPU/Interpreter/MlirModuleInterpreter.cpp:383-405).

Per op (reference file:line):
  conv      MKLConv with a zero bias, then quantizeActivationInt8PerChannelMultiplierAndRShift
            (core/conv.cpp:57-65, 80-104; QuantizationArithmetic.cpp:849-871)
  fc        inner product with the real bias, ReLU, per-tensor qdm requant (core/fullyconnected.cpp:44-91)
  add       copy, scale, sum, ReLU, shift, saturate, pass by pass (core/eltwise.cpp:52-85)
  max pool  MKLPooling (NativeCpuImplementation.h:104-174; padding acts as -inf)
  avg pool  depthwise fp32 conv with an all-ones filter, then the non-qdm rescale (core/pooling.cpp:72-82, 147-154)
  leaky     core/activation.cpp:126-153; clip core/clip.cpp:29-40; upsample core/upsample.cpp:20-41;
  concat    core/concat.cpp:34-90
Under the fp32 guard (every partial sum below 2^24) the results equal the integer oracle's byte
for byte, which tests/test_oracle_dataflow.py checks.
"""
import numpy as np
import torch
import torch.nn.functional as F


def _f32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))


def _saturate_int8(f):
    """saturateInt8 (QuantizationArithmetic.cpp:301-334): floor(f + 0.5) with a double add, clamp"""
    return torch.clamp(torch.floor(f.double() + 0.5), -128, 127).float()


def _srdhm(a, b):
    """SaturatingRoundingDoublingHighMul (:501-509): nudge, then a division truncating toward zero"""
    ab = a.to(torch.int64) * b.to(torch.int64)
    nudge = torch.where(ab >= 0, torch.full_like(ab, 1 << 30), torch.full_like(ab, 1 - (1 << 30)))
    s = ab + nudge
    q = torch.div(s, 1 << 31, rounding_mode="trunc")
    return q.to(torch.int32)


def _rdbp(x, e):
    """RoundingDivideByPOT (:487-499); e is a tensor broadcastable to x"""
    e = e.to(torch.int32)
    mask = (torch.ones_like(e) << e) - 1
    rem = x & mask
    thr = (mask >> 1) + (x < 0).to(torch.int32)
    y = (x >> e) + (rem > thr).to(torch.int32)
    return torch.where(e == 0, x, y)


def _f2u32_i32(t):
    """float parameter -> uint32 at the call -> int32 inside (:863-865, :534)"""
    v = t.to(torch.int64) & 0xFFFFFFFF
    return torch.where(v >= (1 << 31), v - (1 << 32), v).to(torch.int32)


def _requant_qdm(acc_f32, bias, rshift, mult, do_relu, channel_dim):
    """quantizeActivationInt8PerChannelMultiplierAndRShift (:849-871) on a float-stored tensor"""
    shape = [1] * acc_f32.dim()
    shape[channel_dim] = -1
    v = acc_f32.to(torch.int32)
    if bias is not None:
        v = v + bias.to(torch.int32).view(shape)
    x = _srdhm(v, _f2u32_i32(mult).view(shape))
    y = _rdbp(x, _f2u32_i32(rshift).view(shape))
    y = torch.clamp(y, -128, 127)
    if do_relu:
        y = torch.clamp(y, min=0)
    return y.float()


def _mult_rshift_f(x, mult, rshift):
    """the float overload (:518-528): (v * multiplier) / (1 << rshift) evaluated in float"""
    return _saturate_int8((x * float(np.uint32(mult))) / float(1 << int(rshift)))


def run_image(graph, x, keep=None):
    """one N=1 pass; x: float32 [1, C, H, W].  Returns {name: float32 tensor}."""
    vals = {}
    for op in graph.ops:
        ins = [vals[n] for n in op.inputs]
        a, w, t = op.attrs, op.weights, op.type
        if t == "tpu.input":
            y = x
        elif t == "tpu.conv_2d":
            g = int(a["group"])
            filt = _f32(w["filter"]).view(op.shape[1], -1, int(a["kernel_h"]), int(a["kernel_w"]))
            pads = (int(a["padding_l"]), int(a["padding_r"]), int(a["padding_t"]), int(a["padding_b"]))
            xi = F.pad(ins[0], pads) if any(pads) else ins[0]
            acc = F.conv2d(xi, filt, None, (int(a["stride_h"]), int(a["stride_w"])), 0,
                           (int(a["dilation_h"]), int(a["dilation_w"])), g)
            acc = acc[:, :, :op.shape[2], :op.shape[3]]
            bias = _f32(w["bias"]) if int(a["with_bias"]) and "bias" in w else None
            y = _requant_qdm(acc, bias, _f32(w["rshift"]), _f32(w["multiplier"]), bool(a["do_relu"]), 1)
        elif t == "tpu.fully_connected":
            xi = ins[0].reshape(ins[0].shape[0], -1)
            acc = F.linear(xi, _f32(w["filter"]), _f32(w["bias"]) if "bias" in w else None)
            if a.get("do_relu", 0):
                acc = torch.relu(acc)
            y = _requant_qdm(acc, None, _f32(w["rshift"])[:1], _f32(w["multiplier"])[:1], False, 0)
        elif t == "tpu.eltwise_add":
            acc = torch.zeros_like(ins[0])
            for xi, m in zip(ins, w["multiplier"]):
                acc = acc + xi.clone() * float(np.int8(m))
            if a["do_relu"]:
                acc = torch.relu(acc)
            y = _saturate_int8(acc / float(1 << int(w["rshift"][0])))
        elif t == "tpu.pool_max_2d":
            pads = (int(a["padding_l"]), int(a["padding_r"]), int(a["padding_t"]), int(a["padding_b"]))
            xi = F.pad(ins[0], pads, value=float("-inf")) if any(pads) else ins[0]
            y = F.max_pool2d(xi, (int(a["kernel_h"]), int(a["kernel_w"])), (int(a["stride_h"]), int(a["stride_w"])))
            y = y[:, :, :op.shape[2], :op.shape[3]]
        elif t == "tpu.pool_avg_2d":
            c = ins[0].shape[1]
            pads = (int(a["padding_l"]), int(a["padding_r"]), int(a["padding_t"]), int(a["padding_b"]))
            xi = F.pad(ins[0], pads) if any(pads) else ins[0]
            ones = torch.ones(c, 1, int(a["kernel_h"]), int(a["kernel_w"]))
            acc = F.conv2d(xi, ones, None, (int(a["stride_h"]), int(a["stride_w"])), 0, 1, c)
            y = _mult_rshift_f(acc[:, :, :op.shape[2], :op.shape[3]], w["multiplier"][0], w["rshift"][0])
        elif t == "tpu.leaky_relu":
            xi = ins[0]
            pos = _mult_rshift_f(xi, w["multiplier_pos"][0], w["rshift_pos"][0]) if w["multiplier_pos"][0] != 0 else xi
            neg = _mult_rshift_f(xi, w["multiplier_neg"][0], w["rshift_neg"][0])
            y = torch.where(xi > 0, pos, neg)
        elif t == "tpu.clip":
            y = _mult_rshift_f(torch.clamp(ins[0], float(a["min"]), float(a["max"])), w["multiplier"][0], w["rshift"][0])
        elif t == "tpu.upsample":
            y = ins[0].repeat_interleave(int(a["scale_h"]), 2).repeat_interleave(int(a["scale_w"]), 3)
        elif t == "tpu.concat":
            parts = []
            for i, xi in enumerate(ins):
                if "multiplier" in w and "rshift" in w and not (w["multiplier"][i] == 1 and w["rshift"][i] == 0):
                    xi = _mult_rshift_f(xi, w["multiplier"][i], w["rshift"][i])
                parts.append(xi)
            y = torch.cat(parts, int(a["axis"]))
            if a.get("do_relu", 0):
                y = torch.relu(y)
        elif t == "tpu.reshape":
            y = ins[0].reshape((ins[0].shape[0],) + tuple(op.shape[1:]))
        else:
            raise NotImplementedError("data-flow baseline: " + t)
        vals[op.name] = y
    return vals if keep is None else {k: vals[k] for k in keep}


def run(graph, input_data=None, keep=None, images=None):
    """the batch, one image after the other; returns {name: int8 NCHW numpy array}"""
    x = graph.input_op().data if input_data is None else input_data
    n = x.shape[0] if images is None else min(images, x.shape[0])
    names = [op.name for op in graph.ops] if keep is None else list(keep)
    outs = {k: [] for k in names}
    with torch.no_grad():
        for i in range(n):
            v = run_image(graph, _f32(x[i:i + 1]), names)
            for k in names:
                outs[k].append(v[k].numpy())
    return {k: np.concatenate(v, 0).astype(np.int8) for k, v in outs.items()}
