"""Writes a quantized graph in the form the reference's tools read: a TPU-dialect ``.mlir``
in the generic textual syntax plus the ``.npz`` of float32 weight arrays its
``tpu.weight_file`` names (what ``tpuc-opt --tpu-quant`` leaves for ``tpuc-interpreter``:
lib/Dialect/TPU/Backend/test/*.mlir show the syntax, include/tpuc/Dialect/TPU/TPUOps.td
and TPUAttribute.td the attribute names and the param structs).

``module.load(path)`` / ``tpuhip_module_load_mlir`` read such a pair back.
"""
import os
import struct

import numpy as np

from .pymodule import _WEIGHT_OPERANDS

_ELEM = {"INT8": "si8", "UINT8": "ui8", "NONE": "f32", "BF16": "bf16"}

# fields of the param struct attributes (TPUAttribute.td: ConvParam, PoolParam)
_CONV_PARAM = ["kernel_h", "kernel_w", "stride_h", "stride_w", "dilation_h", "dilation_w", "padding_t",
               "padding_b", "padding_l", "padding_r", "group", "is_dw", "with_bias", "pad_value"]
_POOL_PARAM = ["kernel_h", "kernel_w", "padding_t", "padding_b", "padding_l", "padding_r", "pad_value",
               "stride_h", "stride_w", "count_include_pad"]
_BOOLS = {"do_relu", "is_dw", "with_bias", "count_include_pad", "input_transpose", "output_transpose",
          "fused_relu", "do_early_stride", "positive"}
_FLOATS = {"scale", "min", "max", "negative_slope", "const_val", "threshold", "alpha", "beta", "k"}
# numbered float scalars <-> float array attributes
_FLOAT_ARRAYS = {"threshold_parts": 3}
# the activations that become a table lookup in INT8: input, table, mantissa table
_LUT_OPS = {"tpu.sigmoid", "tpu.tanh", "tpu.exp", "tpu.elu", "tpu.swish", "tpu.softplus", "tpu.log", "tpu.pow",
            "tpu.mish", "tpu.sqrt"}
# numbered scalars of an op description <-> array attributes of the dialect
_ARRAYS = {"pads": 8, "crop_offset": 4, "steps": 4, "order": 4, "channel_order": 8, "axes": 4, "ins": 2}
# flag scalars <-> string attributes
_FLAGS = {"mode_edge": ("mode", "edge"), "mode_dcr": ("mode", "DCR")}


def _f32(v):
    """a float attribute the way MLIR prints it: %e when that reads back exactly, else the bits"""
    v = np.float32(v)
    txt = "%.6e" % float(v)
    if np.float32(float(txt)) == v:
        return txt + " : f32"
    return "0x%08X : f32" % struct.unpack("<I", struct.pack("<f", float(v)))[0]


def _scalar(key, v):
    if key in _BOOLS:
        return "true" if v else "false"
    if key in _FLOATS or float(v) != int(v):
        return _f32(v)
    return "%d : i32" % int(v)


def _tensor(shape, elem):
    return "tensor<%sx%s>" % ("x".join(str(int(d)) for d in shape), elem) if len(shape) else "tensor<%s>" % elem


def _attr_dict(op):
    a = dict(op.attrs)
    fields = ['name = "%s"' % op.name]
    if op.type == "tpu.quant":
        src = a.pop("_from", "NONE" if op.quant != "NONE" else "INT8")
        fields += ['from = "%s"' % src, 'to = "%s"' % op.quant]
    else:
        fields.append('quant = {mode = "%s", param_type = "%s", threshold = %s}'
                      % (op.quant, op.param_type, _f32(a.pop("threshold", 0.0))))
    param_keys = _CONV_PARAM if op.type in ("tpu.conv_2d", "tpu.deconv_2d") else \
        _POOL_PARAM if op.type in ("tpu.pool_avg_2d", "tpu.pool_max_2d") else None
    if param_keys is not None:
        p = []
        if op.type in ("tpu.conv_2d", "tpu.deconv_2d"):
            a.setdefault("dilation_h", 1), a.setdefault("dilation_w", 1), a.setdefault("group", 1)
            a.setdefault("is_dw", 0), a.setdefault("with_bias", 1), a.setdefault("pad_value", 0)
            ins_h, ins_w = int(a.pop("ins_h", 0)), int(a.pop("ins_w", 0))
            p.append("ins = [%s]" % ("%d : i32, %d : i32" % (ins_w, ins_h) if ins_h or ins_w else ""))
            p.append('padding = "SAME"')
        else:
            a.setdefault("pad_value", 0), a.setdefault("count_include_pad", 1)
        for k in param_keys:
            if k in a:
                p.append("%s = %s" % (k, _scalar(k, a.pop(k))))
        fields.append("param = {%s}" % ", ".join(sorted(p)))
    for base, n in _ARRAYS.items():
        vals = [a.pop(base + str(i)) for i in range(n) if base + str(i) in a]
        if vals:
            fields.append("%s = [%s]" % (base, ", ".join("%d : i32" % int(v) for v in vals)))
    for base, n in _FLOAT_ARRAYS.items():
        vals = [a.pop(base + str(i)) for i in range(n) if base + str(i) in a]
        if vals:
            fields.append("%s = [%s]" % (base, ", ".join(_f32(v) for v in vals)))
    for flag, (key, text) in _FLAGS.items():
        if a.pop(flag, 0):
            fields.append('%s = "%s"' % (key, text))
    for k in sorted(a):
        if not k.startswith("_"):
            fields.append("%s = %s" % (k, _scalar(k, a[k])))
    return "{%s}" % ", ".join(fields)


def write_mlir(graph, mlir_path, weight_file=None, func_name="tpu_func"):
    """Writes graph to mlir_path and its weights to weight_file (default: beside it, same stem +
    ``_weights.npz``, recorded in the text by base name).  Returns the weight file path."""
    if weight_file is None:
        weight_file = os.path.splitext(mlir_path)[0] + "_weights.npz"
    weights, lines, ids, types = {}, [], {}, {}
    counter = [0]

    def fresh():
        counter[0] += 1
        return "%%%d" % (counter[0] - 1)

    inputs = [op for op in graph.ops if op.type == "tpu.input"]
    args = ["%%arg%d: %s" % (i, _tensor(op.shape, _ELEM[op.quant])) for i, op in enumerate(inputs)]
    wf = fresh()
    lines.append('%s = "tpu.weight_file"() {filename = "%s"} : () -> memref<10xf32>'
                 % (wf, os.path.basename(weight_file)))
    none = fresh()
    lines.append('%s = "tpu.none"() : () -> none' % none)
    n_in = 0
    for op in graph.ops:
        res_t = _tensor(op.shape, _ELEM[op.quant])
        if op.type == "tpu.input":
            me = fresh()
            lines.append('%s = "tpu.input"(%%arg%d) %s : (%s) -> %s' % (me, n_in, _attr_dict(op), res_t, res_t))
            n_in += 1
            ids[op.name], types[op.name] = me, res_t
            continue
        roles = _WEIGHT_OPERANDS.get(op.type)
        if roles is None:
            roles = _WEIGHT_OPERANDS["tpu.lut"] if "table" in op.weights or op.type in _LUT_OPS else []
        opd, opd_t = [ids[s] for s in op.inputs], [types[s] for s in op.inputs]
        for role in roles:
            if role is None or role not in op.weights:
                opd.append(none)
                opd_t.append("none")
                continue
            wname = "%s_%s" % (op.name, role)
            arr = np.ascontiguousarray(op.weights[role], dtype=np.float32)
            weights[wname] = arr
            wid = fresh()
            wt = _tensor(arr.shape, "f32")
            storage = "INT8" if role in ("filter", "table", "slope") else "INT32" if role == "bias" else "UINT32"
            lines.append('%s = "tpu.load_weight"(%s) {name = "%s", storage = "%s"} : (memref<10xf32>) -> %s'
                         % (wid, wf, wname, storage, wt))
            opd.append(wid)
            opd_t.append(wt)
        me = fresh()
        lines.append('%s = "%s"(%s) %s : (%s) -> %s'
                     % (me, op.type, ", ".join(opd), _attr_dict(op), ", ".join(opd_t), res_t))
        ids[op.name], types[op.name] = me, res_t
    outs = list(graph.outputs)
    lines.append("return %s : %s" % (", ".join(ids[o] for o in outs), ", ".join(types[o] for o in outs)))
    res = ", ".join(types[o] for o in outs)
    with open(mlir_path, "w") as f:
        f.write("module {\n  func @%s(%s) -> %s {\n" % (func_name, ", ".join(args),
                                                         res if len(outs) == 1 else "(%s)" % res))
        for line in lines:
            f.write("    %s\n" % line)
        f.write("  }\n}\n")
    if weights:
        np.savez(weight_file, **weights)
    return weight_file
