"""INT8 quantisation arithmetic of the reference's --tpu-quant pass (host only), over the C ABI:
fp32 weights + calibration thresholds -> the float-stored integer operands the INT8 kernels take
(lib/Dialect/TPU/Quantization/QuantizationArithmetic.cpp, QuantizeInt8.cpp)."""
import ctypes as C

import numpy as np

from . import capi

LUT_KINDS = {"sigmoid": 0, "tanh": 1, "exp": 2, "elu": 3, "swish": 4, "softplus": 5, "log": 6, "pow": 7, "mish": 8}


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def quantize_multiplier(m, lib=None):
    """-> (quantized, shift) with m = quantized * 2^(shift - 31)"""
    lib = lib or capi.bind()
    q, s = C.c_int32(0), C.c_int(0)
    capi.check(lib, lib.tpuhip_quantize_multiplier(float(m), C.byref(q), C.byref(s)))
    return q.value, s.value


def find_rshift_and_multiplier(qscale, qdm=False, max_multiplier=127, lib=None):
    lib = lib or capi.bind()
    r, m = C.c_int(0), C.c_uint32(0)
    capi.check(lib, lib.tpuhip_find_rshift_and_multiplier(float(qscale), int(qdm), max_multiplier, C.byref(r),
                                                          C.byref(m)))
    return r.value, m.value


def quantize_conv(filter_, bias, threshold_x, threshold_y, filter_threshold=None, lib=None):
    """filter: (oc, ...) fp32; bias: (oc,) or None -> (filter_q, bias_q or None, rshift, multiplier),
    float32 arrays holding integers, rshift / multiplier per output channel"""
    lib = lib or capi.bind()
    w = _f32(filter_)
    oc, isz = w.shape[0], w.size // w.shape[0]
    b = None if bias is None else _f32(bias)
    ft = None if filter_threshold is None else _f32(filter_threshold)
    wq, bq = np.empty_like(w), (None if b is None else np.empty_like(b))
    rs, mu = np.empty(oc, np.float32), np.empty(oc, np.float32)
    capi.check(lib, lib.tpuhip_quantize_conv_weights(
        w.ctypes.data, None if b is None else b.ctypes.data, oc, isz, threshold_y, threshold_x,
        None if ft is None else ft.ctypes.data, wq.ctypes.data, None if bq is None else bq.ctypes.data,
        rs.ctypes.data, mu.ctypes.data))
    return wq, bq, rs, mu


def quantize_fc(filter_, bias, threshold_x, threshold_y, lib=None):
    """filter: (n, k) or (batch, n, k) -> (filter_q, bias_q or None, rshift, multiplier) per batch"""
    lib = lib or capi.bind()
    w = _f32(filter_)
    batch = 1 if w.ndim == 2 else w.shape[0]
    n, k = w.shape[-2], w.shape[-1]
    b = None if bias is None else _f32(bias)
    wq, bq = np.empty_like(w), (None if b is None else np.empty_like(b))
    rs, mu = np.empty(batch, np.float32), np.empty(batch, np.float32)
    capi.check(lib, lib.tpuhip_quantize_fc_weights(
        w.ctypes.data, None if b is None else b.ctypes.data, batch, n, k, threshold_y, threshold_x,
        wq.ctypes.data, None if bq is None else bq.ctypes.data, rs.ctypes.data, mu.ctypes.data))
    return wq, bq, rs, mu


def quantize_rescale(thresholds_x, threshold_y, coeff=None, divisor=1, lib=None):
    """-> (rshift (1,), multiplier (n_inputs,)) for eltwise add / max / min and average pooling"""
    lib = lib or capi.bind()
    tx = _f32(thresholds_x).reshape(-1)
    cf = None if coeff is None else _f32(coeff).reshape(-1)
    rs, mu = np.empty(1, np.float32), np.empty(tx.size, np.float32)
    capi.check(lib, lib.tpuhip_quantize_rescale(tx.ctypes.data, tx.size, threshold_y,
                                                None if cf is None else cf.ctypes.data, divisor,
                                                rs.ctypes.data, mu.ctypes.data))
    return rs, mu


def quantize_leaky_relu(negative_slope, threshold_x, threshold_y, lib=None):
    """-> dict(rshift_pos, multiplier_pos, rshift_neg, multiplier_neg) of (1,) float32 arrays"""
    lib = lib or capi.bind()
    out = np.empty(4, np.float32)
    capi.check(lib, lib.tpuhip_quantize_leaky_relu(negative_slope, threshold_x, threshold_y, out.ctypes.data))
    keys = ("rshift_pos", "multiplier_pos", "rshift_neg", "multiplier_neg")
    return {k: out[i:i + 1].copy() for i, k in enumerate(keys)}


def quantize_lut_table(kind, threshold_x, threshold_y, scale=1.0, bias=0.0, coeff=0.0, lib=None):
    """-> (256,) float32 table indexed by the two's-complement byte of the int8 input"""
    lib = lib or capi.bind()
    out = np.empty(256, np.float32)
    capi.check(lib, lib.tpuhip_quantize_lut_table(LUT_KINDS[kind], threshold_x, threshold_y, scale, bias, coeff,
                                                  out.ctypes.data))
    return out


def quantize_files(in_mlir, calibration_table, out_mlir, out_weights=None, lib=None):
    """``tpuc-opt --import-calibration-table --calibration-table T --tpu-quant in.mlir -o out.mlir``:
    an fp32 TPU-dialect file + its weight .npz + a calibration table -> the INT8 file ``module.load``
    runs, with its own weight file.  Returns the names of the ops the table had no threshold for."""
    import ctypes as C
    lib = lib or capi.bind()
    args = [str(in_mlir).encode(), str(calibration_table).encode(), str(out_mlir).encode(),
            None if out_weights is None else str(out_weights).encode()]
    buf = C.create_string_buffer(1 << 16)
    need = C.c_size_t(0)
    capi.check(lib, lib.tpuhip_quantize_mlir_files(*args, buf, len(buf), C.byref(need)))
    return [n for n in buf.value.decode().split("\n") if n]
