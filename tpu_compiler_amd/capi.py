"""ctypes binding of the tpuhip C ABI (include/tpuhip.h) plus small numpy
conveniences.  Every call goes to the HIP library; nothing here computes."""
import ctypes as C

import numpy as np

from . import _lib

c_void_pp = C.POINTER(C.c_void_p)


class ConvDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "n", "ic", "ih", "iw", "oc", "oh", "ow", "g", "kh", "kw", "sh", "sw",
        "pt", "pb", "pl", "pr", "dh", "dw", "ins_h", "ins_w", "do_relu", "with_bias",
        "x_cs", "y_cs", "relu_first", "algo")]


class FusedAdd(C.Structure):
    _fields_ = [(k, C.c_int) for k in ("enable", "m_src", "m_conv", "rshift", "do_relu")]


class ConvPost(C.Structure):
    _fields_ = [("lut", C.c_void_p), ("lut_out", C.c_void_p), ("add", FusedAdd),
                ("add_src", C.c_void_p), ("add_out", C.c_void_p),
                ("pool", C.c_void_p), ("pool_out", C.c_void_p)]


class ChainConv(C.Structure):
    _fields_ = [("filter", C.c_void_p), ("bias", C.c_void_p), ("multiplier", C.c_void_p), ("rshift", C.c_void_p)]


class BinaryDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "op", "n", "c", "h", "w", "n0", "c0", "h0", "w0", "n1", "c1", "h1", "w1", "m0", "m1")] + \
        [("multiplier", C.c_int32)] + [(k, C.c_int) for k in ("rshift", "do_relu", "x0_cs", "x1_cs", "y_cs")]


BIN_ADD, BIN_SUB, BIN_MAX, BIN_MIN, BIN_MUL = range(5)


class MoveDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in ("kind", "in_", "ic", "ih", "iw", "on", "oc", "oh", "ow",
                                       "x_cs", "y_cs")] + [("p", C.c_int * 8)]


(MOVE_PAD_CONST, MOVE_PAD_EDGE, MOVE_CROP, MOVE_PERMUTE, MOVE_REORG, MOVE_TILE, MOVE_REVERSE,
 MOVE_SHUFFLE_CHANNEL, MOVE_DEPTH_TO_SPACE, MOVE_SWAP_CHANNEL, MOVE_DILATE,
 MOVE_REFLECTION_PAD) = range(12)


class FcBatchedDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "batch_high", "batch_low", "m", "k", "n", "input_transpose", "output_transpose", "do_relu",
        "x_c", "x_h", "x_w", "x_cs", "y_c", "y_h", "y_w", "y_cs")]


class PoolDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in (
        "n", "c", "ih", "iw", "oh", "ow", "kh", "kw", "sh", "sw", "pt", "pb", "pl", "pr",
        "x_cs", "y_cs")]


ALGO_AUTO, ALGO_DIRECT, ALGO_MFMA, ALGO_DEPTHWISE, ALGO_DEPTHWISE_DOT, ALGO_STEM = 0, 1, 2, 3, 4, 5

# name -> (restype, argtypes); every symbol include/tpuhip.h declares
PROTOTYPES = {
    "tpuhip_ctx_create": (C.c_int, [C.c_int, c_void_pp]),
    "tpuhip_ctx_create_on_stream": (C.c_int, [C.c_int, C.c_void_p, c_void_pp]),
    "tpuhip_ctx_destroy": (C.c_int, [C.c_void_p]),
    "tpuhip_ctx_stream": (C.c_void_p, [C.c_void_p]),
    "tpuhip_ctx_set_autotune": (C.c_int, [C.c_void_p, C.c_int]),
    "tpuhip_last_error": (C.c_char_p, []),
    "tpuhip_version": (C.c_char_p, []),
    "tpuhip_malloc": (C.c_int, [C.c_void_p, C.c_size_t, c_void_pp]),
    "tpuhip_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tpuhip_host_malloc": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "tpuhip_host_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tpuhip_memset": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t]),
    "tpuhip_mem_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "tpuhip_upload": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "tpuhip_download": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "tpuhip_sync": (C.c_int, [C.c_void_p]),
    "tpuhip_event_create": (C.c_int, [C.c_void_p, c_void_pp]),
    "tpuhip_event_destroy": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tpuhip_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tpuhip_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.POINTER(C.c_float)]),
    "tpuhip_ctx_set_kernel_events": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "tpuhip_channel_stride": (C.c_int, [C.c_int]),
    "tpuhip_nchw_to_nhwc_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 5),
    "tpuhip_nhwc_to_nchw_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 5),
    "tpuhip_nchw_f32_to_nhwc_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 5),
    "tpuhip_nhwc_i8_to_nchw_f32": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 5),
    "tpuhip_conv2d_prepack": (C.c_int, [C.c_void_p, C.POINTER(ConvDesc), C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_void_p, c_void_pp]),
    "tpuhip_conv2d_weights_destroy": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tpuhip_conv2d_i8": (C.c_int, [C.c_void_p] * 4),
    "tpuhip_conv2d_algo_name": (C.c_char_p, [C.c_void_p]),
    "tpuhip_conv2d_tile_name": (C.c_char_p, [C.c_int]),
    "tpuhip_conv2d_can_fuse_table": (C.c_int, [C.c_void_p]),
    "tpuhip_conv2d_add_i8": (C.c_int, [C.c_void_p] * 6 + [C.POINTER(FusedAdd)]),
    "tpuhip_conv2d_post_i8": (C.c_int, [C.c_void_p] * 4 + [C.POINTER(ConvPost)]),
    "tpuhip_lut_per_channel_i8": (C.c_int, [C.c_void_p] * 4 + [C.c_size_t, C.c_int, C.c_int]),
    "tpuhip_prelu_tables": (C.c_int, [C.POINTER(C.c_float), C.c_int, C.c_uint32, C.c_uint32, C.c_uint32,
                                      C.POINTER(C.c_int8)]),
    "tpuhip_quant_f32_to_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 5 + [C.c_float]),
    "tpuhip_dequant_i8_to_f32": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 5 + [C.c_float]),
    "tpuhip_permute_flat_i8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "tpuhip_move_i8": (C.c_int, [C.c_void_p, C.POINTER(MoveDesc), C.c_void_p, C.c_void_p]),
    "tpuhip_binary_i8": (C.c_int, [C.c_void_p, C.POINTER(BinaryDesc)] + [C.c_void_p] * 3),
    "tpuhip_conv2d_can_fuse_pool": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(PoolDesc)]),
    "tpuhip_fc_prepack": (C.c_int, [C.c_void_p] + [C.c_int] * 6 + [C.c_void_p, C.c_void_p,
                                                                   C.c_int32, C.c_int32,
                                                                   c_void_pp]),
    "tpuhip_fc_i8": (C.c_int, [C.c_void_p] * 4),
    "tpuhip_fc_i8_noalloc": (C.c_int, [C.c_void_p] * 4),
    "tpuhip_fc_batched_prepack": (C.c_int, [C.c_void_p, C.POINTER(FcBatchedDesc)] + [C.c_void_p] * 4 +
                                  [c_void_pp]),
    "tpuhip_fc_batched_destroy": (C.c_int, [C.c_void_p] * 2),
    "tpuhip_fc_batched_i8": (C.c_int, [C.c_void_p] * 4),
    "tpuhip_eltwise_add_i8": (C.c_int, [C.c_void_p, c_void_pp, C.c_int, C.c_void_p, C.c_int,
                                        C.c_int, C.c_void_p, C.c_size_t]),
    "tpuhip_pool_max_i8": (C.c_int, [C.c_void_p, C.POINTER(PoolDesc), C.c_void_p, C.c_void_p]),
    "tpuhip_pool_avg_i8": (C.c_int, [C.c_void_p, C.POINTER(PoolDesc), C.c_void_p, C.c_void_p,
                                     C.c_uint32, C.c_uint32]),
    "tpuhip_lut_i8": (C.c_int, [C.c_void_p] * 4 + [C.c_size_t, C.c_int, C.c_int]),
    "tpuhip_leaky_relu_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_size_t, C.c_int, C.c_int] +
                             [C.c_uint32] * 4),
    "tpuhip_leaky_relu_table": (C.c_int, [C.c_uint32] * 4 + [C.c_void_p]),
    "tpuhip_clip_table": (C.c_int, [C.c_float, C.c_float, C.c_uint32, C.c_uint32, C.c_void_p]),
    "tpuhip_relu_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_size_t]),
    "tpuhip_upsample_nearest_i8": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 8),
    "tpuhip_concat_i8": (C.c_int, [C.c_void_p, c_void_pp, C.c_int, C.c_void_p, C.c_void_p,
                                   C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int]),
}


class OpDescC(C.Structure):
    _fields_ = [("type", C.c_char_p), ("name", C.c_char_p), ("quant", C.c_char_p),
                ("param_type", C.c_char_p), ("ndim", C.c_int), ("shape", C.POINTER(C.c_int64)),
                ("n_operands", C.c_int), ("operands", C.POINTER(C.c_char_p)),
                ("n_attrs", C.c_int), ("attr_keys", C.POINTER(C.c_char_p)),
                ("attr_values", C.POINTER(C.c_double))]


PROTOTYPES.update({
    "tpuhip_module_create": (C.c_int, [C.c_int, C.c_int, c_void_pp]),
    "tpuhip_module_destroy": (C.c_int, [C.c_void_p]),
    "tpuhip_module_set_weight": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t]),
    "tpuhip_module_clear_ops": (C.c_int, [C.c_void_p]),
    "tpuhip_module_add_op": (C.c_int, [C.c_void_p, C.POINTER(OpDescC)]),
    "tpuhip_module_set_returns": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.c_int]),
    "tpuhip_module_load": (C.c_int, [C.c_void_p, C.c_char_p]),
    "tpuhip_module_set_tensor": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t,
                                           C.c_int]),
    "tpuhip_module_set_tensor_i8": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.c_int]),
    "tpuhip_module_get_tensor": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t,
                                           C.c_int]),
    "tpuhip_module_get_tensor_i8": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t,
                                              C.c_int]),
    "tpuhip_module_invoke": (C.c_int, [C.c_void_p, C.c_int]),
    "tpuhip_module_invoke_to": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int]),
    "tpuhip_module_fast_invoke_all_batch": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int]),
    "tpuhip_module_sync": (C.c_int, [C.c_void_p]),
    "tpuhip_module_tensor_shape": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64),
                                             C.POINTER(C.c_int)]),
    "tpuhip_module_tensor_dtype": (C.c_char_p, [C.c_void_p, C.c_char_p]),
    "tpuhip_module_num_tensors": (C.c_int, [C.c_void_p]),
    "tpuhip_module_tensor_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "tpuhip_module_num_inputs": (C.c_int, [C.c_void_p]),
    "tpuhip_module_input_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "tpuhip_module_num_outputs": (C.c_int, [C.c_void_p]),
    "tpuhip_module_output_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "tpuhip_module_num_kernels": (C.c_int, [C.c_void_p]),
    "tpuhip_module_kernel_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "tpuhip_module_kernel_algo": (C.c_char_p, [C.c_void_p, C.c_int]),
    "tpuhip_module_time_kernels": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_float),
                                             C.c_int]),
    "tpuhip_module_ctx": (C.c_void_p, [C.c_void_p]),
    "tpuhip_module_set_option": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int]),
    "tpuhip_conv2d_prepack_pair": (C.c_int, [C.c_void_p, C.POINTER(ConvDesc), C.POINTER(ConvDesc), C.c_void_p,
                                             C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                             C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]),
    "tpuhip_conv2d_pair_i8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "tpuhip_conv2d_can_chain": (C.c_int, [C.POINTER(ConvDesc), C.POINTER(ConvDesc)]),
    "tpuhip_conv2d_chain_prepack": (C.c_int, [C.c_void_p, C.POINTER(ConvDesc), C.POINTER(ConvDesc), C.c_void_p,
                                              C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                              C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]),
    "tpuhip_conv2d_chain_destroy": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tpuhip_conv2d_chain_i8": (C.c_int, [C.c_void_p] * 6 + [C.POINTER(FusedAdd), C.c_void_p]),
    "tpuhip_conv2d_set_input_stride": (C.c_int, [C.c_void_p, C.c_int]),
    "tpuhip_conv2d_chain_kind": (C.c_int, [C.POINTER(ConvDesc), C.POINTER(ConvDesc)]),
    "tpuhip_conv2d_chain_post_i8": (C.c_int, [C.c_void_p] * 4 + [C.POINTER(ConvPost), C.c_void_p, C.POINTER(ConvPost)]),
    "tpuhip_conv2d_can_chain3": (C.c_int, [C.POINTER(ConvDesc)] * 3),
    "tpuhip_conv2d_chain3_prepack": (C.c_int, [C.c_void_p] + [C.POINTER(ConvDesc)] * 3 + [C.POINTER(ChainConv)] * 3 + [c_void_pp]),
    "tpuhip_conv2d_chain3_i8": (C.c_int, [C.c_void_p] * 4 + [C.POINTER(ConvPost)]),
    "tpuhip_conv2d_chain_name": (C.c_char_p, [C.c_void_p]),
    "tpuhip_conv2d_chain_variant_name": (C.c_char_p, [C.c_int]),
    "tpuhip_module_load_mlir": (C.c_int, [C.c_void_p, C.c_char_p, C.c_char_p]),
    "tpuhip_module_weight_file": (C.c_char_p, [C.c_void_p]),
    "tpuhip_module_num_ops": (C.c_int, [C.c_void_p]),
    "tpuhip_module_op_info": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_char_p),
                                        C.POINTER(C.c_char_p), C.POINTER(C.c_char_p)]),
    "tpuhip_module_interpret_files": (C.c_int, [C.c_void_p, C.c_char_p, C.c_char_p, C.c_char_p,
                                                C.c_char_p]),
    "tpuhip_mlir_describe": (C.c_int, [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]),
    "tpuhip_npz_open": (C.c_int, [C.c_char_p, C.c_int, C.POINTER(C.c_void_p)]),
    "tpuhip_npz_close": (C.c_int, [C.c_void_p]),
    "tpuhip_npz_count": (C.c_int, [C.c_void_p]),
    "tpuhip_npz_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "tpuhip_npz_info": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64), C.POINTER(C.c_int),
                                  C.POINTER(C.c_char), C.POINTER(C.c_int)]),
    "tpuhip_npz_read_f32": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t]),
    "tpuhip_npz_add_f32": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.POINTER(C.c_int64), C.c_int]),
    "tpuhip_npz_delete": (C.c_int, [C.c_void_p, C.c_char_p]),
    "tpuhip_npz_keep": (C.c_int, [C.c_void_p]),
    "tpuhip_quantize_multiplier": (C.c_int, [C.c_double, C.POINTER(C.c_int32), C.POINTER(C.c_int)]),
    "tpuhip_find_rshift_and_multiplier": (C.c_int, [C.c_double, C.c_int, C.c_uint32, C.POINTER(C.c_int),
                                                    C.POINTER(C.c_uint32)]),
    "tpuhip_quantize_conv_weights": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_float,
                                               C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_void_p]),
    "tpuhip_quantize_fc_weights": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                             C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p,
                                             C.c_void_p]),
    "tpuhip_quantize_rescale": (C.c_int, [C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_int, C.c_void_p,
                                          C.c_void_p]),
    "tpuhip_quantize_leaky_relu": (C.c_int, [C.c_float, C.c_float, C.c_float, C.c_void_p]),
    "tpuhip_reduce_i8": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.POINTER(C.c_int), C.c_int,
                                   C.POINTER(C.c_int), C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint32]),
    "tpuhip_lrn_i8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int,
                                C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]),
    "tpuhip_quantize_mlir_files": (C.c_int, [C.c_char_p, C.c_char_p, C.c_char_p, C.c_char_p, C.c_char_p,
                                             C.c_size_t, C.POINTER(C.c_size_t)]),
    "tpuhip_quantize_lut_table": (C.c_int, [C.c_int, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float,
                                            C.c_void_p]),
})


class TpuHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("tpuhip status %d: %s" % (status, message))
        self.status = status


def bind(lib=None, prototypes=None):
    lib = lib or _lib.load()
    for name, (res, args) in (prototypes or PROTOTYPES).items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def check(lib, status):
    if status != 0:
        raise TpuHipError(status, lib.tpuhip_last_error().decode("utf-8", "replace"))


def mlir_describe(path, lib=None):
    """what the reader understood of a TPU-dialect .mlir file, one line per weight / op / return
    (parses only: no GPU, no weight file)"""
    lib = lib or bind()
    need = C.c_size_t(0)
    check(lib, lib.tpuhip_mlir_describe(str(path).encode(), None, 0, C.byref(need)))
    buf = C.create_string_buffer(need.value)
    check(lib, lib.tpuhip_mlir_describe(str(path).encode(), buf, need.value, None))
    return buf.value.decode()


class TensorFile:
    """include/tpuc/Support/TensorFile.h: an .npz of arrays keyed by name.  mode "r" = read only,
    "w" = start empty, "a" = read what exists and allow changes; keep() writes the file."""

    def __init__(self, filename, mode="r", lib=None):
        self.lib = lib or bind()
        self.h = C.c_void_p()
        check(self.lib, self.lib.tpuhip_npz_open(str(filename).encode(), {"r": 0, "w": 1, "a": 2}[mode],
                                                 C.byref(self.h)))

    def close(self):
        if self.h:
            self.lib.tpuhip_npz_close(self.h)
            self.h = None

    def names(self):
        # member names are bytes in the archive: anything that is not UTF-8 survives the round trip
        return [self.lib.tpuhip_npz_name(self.h, i).decode("utf-8", "surrogateescape")
                for i in range(self.lib.tpuhip_npz_count(self.h))]

    def info(self, name):
        dims, nd, kind, ws = (C.c_int64 * 8)(), C.c_int(0), C.c_char(b"?"), C.c_int(0)
        check(self.lib, self.lib.tpuhip_npz_info(self.h, name.encode("utf-8", "surrogateescape"), dims, C.byref(nd), C.byref(kind),
                                                 C.byref(ws)))
        return tuple(dims[i] for i in range(nd.value)), kind.value.decode(), ws.value

    def read(self, name):
        shape, _, _ = self.info(name)
        out = np.empty(shape, np.float32)
        check(self.lib, self.lib.tpuhip_npz_read_f32(self.h, name.encode("utf-8", "surrogateescape"), out.ctypes.data, out.size))
        return out

    def add(self, name, array):
        a = np.asarray(array, dtype=np.float32, order="C")    # keeps a 0-d array 0-d
        dims = (C.c_int64 * max(a.ndim, 1))(*a.shape)
        check(self.lib, self.lib.tpuhip_npz_add_f32(self.h, name.encode("utf-8", "surrogateescape"), a.ctypes.data, dims, a.ndim))

    def delete(self, name):
        check(self.lib, self.lib.tpuhip_npz_delete(self.h, name.encode("utf-8", "surrogateescape")))

    def keep(self):
        check(self.lib, self.lib.tpuhip_npz_keep(self.h))


def channel_stride(c):
    return (c + 15) // 16 * 16


class DeviceTensor:
    """An int8 channels-last tensor in HBM: logical NCHW shape, channel stride cs."""

    def __init__(self, ctx, shape, cs=None, ptr=None, owner=True):
        self.ctx = ctx
        self.shape = tuple(int(v) for v in shape)
        n, c, h, w = self.shape
        self.cs = cs or channel_stride(c)
        if self.cs < c or (self.cs % 16 and self.cs != 4):
            raise TpuHipError(2, "a channel stride is 4 or a multiple of 16 and covers the channels (%d for %d)"
                              % (self.cs, c))
        self.nbytes = n * h * w * self.cs
        self._owner = owner and ptr is None
        self.ptr = ptr if ptr is not None else ctx.malloc(self.nbytes)

    @property
    def pixels(self):
        n, _, h, w = self.shape
        return n * h * w

    def free(self):
        if self._owner and self.ptr:
            self.ctx.free(self.ptr)
            self.ptr = None


class Context:
    """One tpuhip context (one HIP stream) with numpy conveniences."""

    def __init__(self, device=0):
        self.lib = bind()
        h = C.c_void_p()
        check(self.lib, self.lib.tpuhip_ctx_create(device, C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            self.lib.tpuhip_ctx_destroy(self.h)
            self.h = None

    def _ck(self, status):
        check(self.lib, status)

    # -- memory -----------------------------------------------------------
    def malloc(self, nbytes):
        p = C.c_void_p()
        self._ck(self.lib.tpuhip_malloc(self.h, max(int(nbytes), 1), C.byref(p)))
        return p.value

    def free(self, ptr):
        self._ck(self.lib.tpuhip_free(self.h, ptr))

    def upload(self, ptr, arr):
        arr = np.ascontiguousarray(arr)
        self._ck(self.lib.tpuhip_upload(self.h, ptr, arr.ctypes.data, arr.nbytes))

    def download(self, ptr, shape, dtype):
        out = np.empty(shape, dtype)
        self._ck(self.lib.tpuhip_download(self.h, out.ctypes.data, ptr, out.nbytes))
        return out

    def sync(self):
        self._ck(self.lib.tpuhip_sync(self.h))

    def mem_info(self):
        """(free, total) device bytes as the library's HIP runtime sees them"""
        free, total = C.c_size_t(), C.c_size_t()
        self._ck(self.lib.tpuhip_mem_info(self.h, C.byref(free), C.byref(total)))
        return free.value, total.value

    # -- events ------------------------------------------------------------
    def event(self):
        e = C.c_void_p()
        self._ck(self.lib.tpuhip_event_create(self.h, C.byref(e)))
        return e.value

    def record(self, ev):
        self._ck(self.lib.tpuhip_event_record(self.h, ev))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        self._ck(self.lib.tpuhip_event_elapsed_ms(self.h, start, stop, C.byref(ms)))
        return ms.value

    # -- tensors -------------------------------------------------------------
    def tensor(self, shape, cs=None):
        return DeviceTensor(self, shape, cs)

    def from_nchw(self, arr, cs=None):
        """int8 NCHW numpy array -> channels-last device tensor (conversion on the GPU)."""
        arr = np.ascontiguousarray(arr)
        assert arr.dtype == np.int8 and arr.ndim == 4
        t = DeviceTensor(self, arr.shape, cs)
        tmp = self.malloc(arr.nbytes)
        try:
            self.upload(tmp, arr)
            n, c, h, w = arr.shape
            self._ck(self.lib.tpuhip_nchw_to_nhwc_i8(self.h, tmp, t.ptr, n, c, h, w, t.cs))
            self.sync()
        finally:
            self.free(tmp)
        return t

    def to_nchw(self, t):
        n, c, h, w = t.shape
        tmp = self.malloc(n * c * h * w)
        try:
            self._ck(self.lib.tpuhip_nhwc_to_nchw_i8(self.h, t.ptr, tmp, n, c, h, w, t.cs))
            return self.download(tmp, t.shape, np.int8)
        finally:
            self.free(tmp)

    def raw(self, t):
        """the channels-last bytes, pad channels included"""
        n, c, h, w = t.shape
        return self.download(t.ptr, (n, h, w, t.cs), np.int8)

    # -- ops -------------------------------------------------------------------
    def conv_prepack(self, desc, filt, bias, mult, rshift):
        filt = np.ascontiguousarray(filt, dtype=np.int8)
        mult = np.ascontiguousarray(mult, dtype=np.int32)
        rshift = np.ascontiguousarray(rshift, dtype=np.int32)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        w = C.c_void_p()
        self._ck(self.lib.tpuhip_conv2d_prepack(
            self.h, C.byref(desc), filt.ctypes.data, None if b is None else b.ctypes.data,
            mult.ctypes.data, rshift.ctypes.data, C.byref(w)))
        return w.value

    def lrn(self, x, y, local_size, sqr_lut, power_lut, sum_rshift, lrn_rshift, quant0, quant1):
        sq = np.ascontiguousarray(sqr_lut, dtype=np.uint8)
        pw = np.ascontiguousarray(power_lut, dtype=np.uint8)
        assert sq.size == 256 and pw.size == 256
        n, c, h, w = x.shape
        self._ck(self.lib.tpuhip_lrn_i8(self.h, x.ptr, y.ptr, n * h * w, c, x.cs, int(local_size),
                                        sq.ctypes.data, pw.ctypes.data, int(sum_rshift), int(lrn_rshift),
                                        int(quant0), int(quant1)))

    def conv_prepack_pair(self, desc_a, desc_b, a, b):
        """a, b: (filter int8, bias int32 or None, multiplier int32, rshift int32) of two convs over
        the same input with the same window geometry -> one handle for conv_pair"""
        keep, ptrs = [], []
        for filt, bias, mult, rshift in (a, b):
            arrs = [np.ascontiguousarray(filt, dtype=np.int8),
                    None if bias is None else np.ascontiguousarray(bias, dtype=np.int32),
                    np.ascontiguousarray(mult, dtype=np.int32), np.ascontiguousarray(rshift, dtype=np.int32)]
            keep += arrs
            ptrs += [None if x is None else x.ctypes.data for x in arrs]
        w = C.c_void_p()
        self._ck(self.lib.tpuhip_conv2d_prepack_pair(self.h, C.byref(desc_a), C.byref(desc_b), *ptrs,
                                                     C.byref(w)))
        return w.value

    def conv_pair(self, w, x, y_a, y_b):
        self._ck(self.lib.tpuhip_conv2d_pair_i8(self.h, w, x.ptr, y_a.ptr, y_b.ptr))

    def conv_can_chain(self, desc_a, desc_b):
        return bool(self.lib.tpuhip_conv2d_can_chain(C.byref(desc_a), C.byref(desc_b)))

    def conv_chain_prepack(self, desc_a, desc_b, a, b):
        """a, b: (filter int8, bias int32 or None, multiplier int32, rshift int32) of two pointwise convs,
        the second reading what the first (or the add behind it) produces -> one handle for conv_chain"""
        keep, ptrs = [], []
        for filt, bias, mult, rshift in (a, b):
            arrs = [np.ascontiguousarray(filt, dtype=np.int8),
                    None if bias is None else np.ascontiguousarray(bias, dtype=np.int32),
                    np.ascontiguousarray(mult, dtype=np.int32), np.ascontiguousarray(rshift, dtype=np.int32)]
            keep += arrs
            ptrs += [None if x is None else x.ctypes.data for x in arrs]
        w = C.c_void_p()
        self._ck(self.lib.tpuhip_conv2d_chain_prepack(self.h, C.byref(desc_a), C.byref(desc_b), *ptrs,
                                                      C.byref(w)))
        return w.value

    def conv_chain(self, ch, x, y_b, y_a=None, add=None):
        """add = (src, out or None, m_src, m_conv, rshift, relu)"""
        f = None
        src = out = None
        if add is not None:
            src, out, m_src, m_conv, rshift, relu = add
            f = FusedAdd(1, int(m_src), int(m_conv), int(rshift), int(relu))
        self._ck(self.lib.tpuhip_conv2d_chain_i8(
            self.h, ch, x.ptr, None if y_a is None else y_a.ptr, None if src is None else src.ptr,
            None if out is None else out.ptr, None if f is None else C.byref(f), y_b.ptr))

    def conv_chain_kind(self, desc_a, desc_b):
        """0: no chain; 1: two pointwise convs; 2: a depthwise conv and the pointwise conv behind it"""
        return int(self.lib.tpuhip_conv2d_chain_kind(C.byref(desc_a), C.byref(desc_b)))

    def conv_chain_post(self, ch, x, y_b=None, y_a=None, table_a=None, lut_out_a=None, add_a=None, add_b=None):
        """the general chain call: a table and / or an add = (src, out or None, m_src, m_conv, rshift, relu)
        behind conv A, an add behind conv B, as far as the chain's kind takes them"""
        pa, pb = ConvPost(), ConvPost()
        keep = None
        if table_a is not None:
            keep = np.ascontiguousarray(table_a, dtype=np.int8)
            assert keep.size == 256
            pa.lut = keep.ctypes.data
            pa.lut_out = None if lut_out_a is None else lut_out_a.ptr
        for post, add in ((pa, add_a), (pb, add_b)):
            if add is not None:
                src, out, m_src, m_conv, rshift, relu = add
                post.add = FusedAdd(1, int(m_src), int(m_conv), int(rshift), int(relu))
                post.add_src = src.ptr
                post.add_out = None if out is None else out.ptr
        self._ck(self.lib.tpuhip_conv2d_chain_post_i8(
            self.h, ch, x.ptr, None if y_a is None else y_a.ptr, C.byref(pa),
            None if y_b is None else y_b.ptr, C.byref(pb)))

    def conv_can_chain3(self, desc_e, desc_d, desc_p):
        return bool(self.lib.tpuhip_conv2d_can_chain3(C.byref(desc_e), C.byref(desc_d), C.byref(desc_p)))

    def conv_chain3_prepack(self, desc_e, desc_d, desc_p, e, d, p):
        """e, d, p: (filter int8, bias int32 or None, multiplier int32, rshift int32) of the 1x1 expansion, the
        depthwise conv and the 1x1 projection of an inverted-residual block -> one handle for conv_chain3"""
        keep, packs = [], []
        for filt, bias, mult, rshift in (e, d, p):
            arrs = [np.ascontiguousarray(filt, dtype=np.int8),
                    None if bias is None else np.ascontiguousarray(bias, dtype=np.int32),
                    np.ascontiguousarray(mult, dtype=np.int32), np.ascontiguousarray(rshift, dtype=np.int32)]
            keep += arrs
            packs.append(ChainConv(*[None if x is None else x.ctypes.data for x in arrs]))
        w = C.c_void_p()
        self._ck(self.lib.tpuhip_conv2d_chain3_prepack(self.h, C.byref(desc_e), C.byref(desc_d), C.byref(desc_p),
                                                       C.byref(packs[0]), C.byref(packs[1]), C.byref(packs[2]),
                                                       C.byref(w)))
        return w.value

    def conv_chain3(self, ch, x, y=None, add=None):
        """add = (src, out, m_src, m_conv, rshift, relu) behind the projection"""
        post = ConvPost()
        if add is not None:
            src, out, m_src, m_conv, rshift, relu = add
            post.add = FusedAdd(1, int(m_src), int(m_conv), int(rshift), int(relu))
            post.add_src, post.add_out = src.ptr, out.ptr
        self._ck(self.lib.tpuhip_conv2d_chain3_i8(self.h, ch, x.ptr, None if y is None else y.ptr, C.byref(post)))

    def conv_chain_destroy(self, ch):
        self._ck(self.lib.tpuhip_conv2d_chain_destroy(self.h, ch))

    def conv_chain_name(self, ch):
        return self.lib.tpuhip_conv2d_chain_name(ch).decode()

    def fc_prepack(self, m, k, n, x_cs, y_cs, do_relu, filt, bias, mult, rshift):
        filt = np.ascontiguousarray(filt, dtype=np.int8)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        w = C.c_void_p()
        self._ck(self.lib.tpuhip_fc_prepack(
            self.h, m, k, n, x_cs, y_cs, int(do_relu), filt.ctypes.data,
            None if b is None else b.ctypes.data, int(mult), int(rshift), C.byref(w)))
        return w.value

    def fc(self, w, x, y, noalloc=False):
        f = self.lib.tpuhip_fc_i8_noalloc if noalloc else self.lib.tpuhip_fc_i8
        self._ck(f(self.h, w, x.ptr, y.ptr))

    def fc_batched_prepack(self, desc, filt, bias, mult, rshift):
        filt = np.ascontiguousarray(filt, dtype=np.int8)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        mu = np.ascontiguousarray(mult, dtype=np.int32)
        rs = np.ascontiguousarray(rshift, dtype=np.int32)
        w = C.c_void_p()
        self._ck(self.lib.tpuhip_fc_batched_prepack(
            self.h, C.byref(desc), filt.ctypes.data, None if b is None else b.ctypes.data,
            mu.ctypes.data, rs.ctypes.data, C.byref(w)))
        return w.value

    def fc_batched(self, w, x, y):
        self._ck(self.lib.tpuhip_fc_batched_i8(self.h, w, x.ptr, y.ptr))

    def fc_batched_destroy(self, w):
        self._ck(self.lib.tpuhip_fc_batched_destroy(self.h, w))

    def conv_weights_destroy(self, w):
        self._ck(self.lib.tpuhip_conv2d_weights_destroy(self.h, w))

    def conv(self, w, x, y):
        self._ck(self.lib.tpuhip_conv2d_i8(self.h, w, x.ptr if hasattr(x, "ptr") else x,
                                           y.ptr if hasattr(y, "ptr") else y))

    def conv_add(self, w, x, y, add_src, add_out, m_src, m_conv, rshift, do_relu):
        f = FusedAdd(1, int(m_src), int(m_conv), int(rshift), int(do_relu))
        self._ck(self.lib.tpuhip_conv2d_add_i8(self.h, w, x.ptr, None if y is None else y.ptr,
                                               add_src.ptr, add_out.ptr, C.byref(f)))

    def conv_can_fuse_pool(self, w, pool_desc):
        return bool(self.lib.tpuhip_conv2d_can_fuse_pool(self.h, w, C.byref(pool_desc)))

    def conv_post(self, w, x, y=None, table=None, lut_out=None, add=None, pool=None):
        """conv, then the optional table, then the optional add = (src, out, m_src, m_conv, rshift, relu);
        or conv, then the max pool = (PoolDesc, out) in the same launch"""
        p = ConvPost()
        t = None
        if pool is not None:
            p.pool = C.addressof(pool[0])
            p.pool_out = pool[1].ptr
        if table is not None:
            t = np.ascontiguousarray(table, dtype=np.int8)
            assert t.size == 256
            p.lut = t.ctypes.data
            p.lut_out = None if lut_out is None else lut_out.ptr
        if add is not None:
            src, out, m_src, m_conv, rshift, relu = add
            p.add = FusedAdd(1, int(m_src), int(m_conv), int(rshift), int(relu))
            p.add_src, p.add_out = src.ptr, out.ptr
        self._ck(self.lib.tpuhip_conv2d_post_i8(self.h, w, x.ptr, None if y is None else y.ptr,
                                                C.byref(p)))

    def conv_set_input_stride(self, w, x_cs):
        self._ck(self.lib.tpuhip_conv2d_set_input_stride(w, int(x_cs)))

    def conv_algo_name(self, w):
        return self.lib.tpuhip_conv2d_algo_name(w).decode()

    def eltwise_add(self, xs, mult, rshift, do_relu, y):
        ptrs = (C.c_void_p * len(xs))(*[t.ptr for t in xs])
        m = np.ascontiguousarray(mult, dtype=np.int8)
        self._ck(self.lib.tpuhip_eltwise_add_i8(self.h, ptrs, len(xs), m.ctypes.data, int(rshift),
                                                int(do_relu), y.ptr, y.nbytes))

    def move(self, kind, x, y, params):
        p = (C.c_int * 8)(*(list(params) + [0] * (8 - len(params))))
        d = MoveDesc(kind, *x.shape, *y.shape, x.cs, y.cs, p)
        self._ck(self.lib.tpuhip_move_i8(self.h, C.byref(d), x.ptr, y.ptr))

    def prelu(self, x, y, slope, rshift_pos, multiplier_pos, rshift_neg):
        c = x.shape[1]
        sl = np.ascontiguousarray(slope, dtype=np.float32)
        tables = np.empty(c * 256, np.int8)
        self._ck(self.lib.tpuhip_prelu_tables(sl.ctypes.data_as(C.POINTER(C.c_float)), c,
                                              int(rshift_pos), int(multiplier_pos), int(rshift_neg),
                                              tables.ctypes.data_as(C.POINTER(C.c_int8))))
        dev = self.malloc(tables.nbytes)
        self.upload(dev, tables)
        self._ck(self.lib.tpuhip_lut_per_channel_i8(self.h, x.ptr, y.ptr, dev, x.pixels, c, x.cs))
        self.sync()
        self.free(dev)

    def binary(self, op, x0, x1, y, m0=1, m1=1, multiplier=0, rshift=0, do_relu=False):
        """x0, x1, y: device tensors made by tensor()/from_nchw() (logical NCHW shapes)"""
        s0, s1, so = x0.shape, x1.shape, y.shape
        d = BinaryDesc(op, so[0], so[1], so[2], so[3], s0[0], s0[1], s0[2], s0[3],
                       s1[0], s1[1], s1[2], s1[3], int(m0), int(m1), int(multiplier), int(rshift),
                       int(do_relu), x0.cs, x1.cs, y.cs)
        self._ck(self.lib.tpuhip_binary_i8(self.h, C.byref(d), x0.ptr, x1.ptr, y.ptr))

    def pool_max(self, d, x, y):
        self._ck(self.lib.tpuhip_pool_max_i8(self.h, C.byref(d), x.ptr, y.ptr))

    def pool_avg(self, d, x, y, mult, rshift):
        self._ck(self.lib.tpuhip_pool_avg_i8(self.h, C.byref(d), x.ptr, y.ptr, int(mult),
                                             int(rshift)))

    def lut(self, x, y, table):
        t = np.ascontiguousarray(table, dtype=np.int8)
        assert t.size == 256
        self._ck(self.lib.tpuhip_lut_i8(self.h, x.ptr, y.ptr, t.ctypes.data, x.pixels,
                                        x.shape[1], x.cs))

    def leaky_relu(self, x, y, rp, mp, rn, mn):
        self._ck(self.lib.tpuhip_leaky_relu_i8(self.h, x.ptr, y.ptr, x.pixels, x.shape[1], x.cs,
                                               int(rp), int(mp), int(rn), int(mn)))

    def leaky_relu_table(self, rp, mp, rn, mn):
        t = np.empty(256, np.int8)
        self._ck(self.lib.tpuhip_leaky_relu_table(int(rp), int(mp), int(rn), int(mn),
                                                  t.ctypes.data))
        return t

    def clip_table(self, lo, hi, rshift, mult):
        t = np.empty(256, np.int8)
        self._ck(self.lib.tpuhip_clip_table(float(lo), float(hi), int(rshift), int(mult),
                                            t.ctypes.data))
        return t

    def relu(self, x, y):
        self._ck(self.lib.tpuhip_relu_i8(self.h, x.ptr, y.ptr, x.nbytes))

    def upsample(self, x, y, sh, sw):
        n, c, h, w = x.shape
        self._ck(self.lib.tpuhip_upsample_nearest_i8(self.h, x.ptr, y.ptr, n, c, h, w, sh, sw,
                                                     x.cs, y.cs))

    def concat(self, xs, axis, y, rshift=None, mult=None, do_relu=False):
        ptrs = (C.c_void_p * len(xs))(*[t.ptr for t in xs])
        dims = np.ascontiguousarray(np.array([t.shape for t in xs], dtype=np.int32))
        cs = np.ascontiguousarray(np.array([t.cs for t in xs], dtype=np.int32))
        r = None if rshift is None else np.ascontiguousarray(rshift, dtype=np.uint32)
        m = None if mult is None else np.ascontiguousarray(mult, dtype=np.uint32)
        self._ck(self.lib.tpuhip_concat_i8(
            self.h, ptrs, len(xs), dims.ctypes.data, cs.ctypes.data, axis,
            None if r is None else r.ctypes.data, None if m is None else m.ctypes.data,
            int(do_relu), y.ptr, y.cs))
