"""`module`: the Python face of the interpreter, shaped like the reference's
pymlir.module (bindings/python/pymlir.cpp:87-311): load / run / set_tensor /
get_tensor / invoke / invoke_to / get_all_tensor / op_info / get_input_details /
get_output_details.  Where pymlir.load parses an .mlir file, `load` takes a
`graphs.Graph` (ops in program order with their float-stored weights).

Tensors cross this API as float32 NCHW arrays holding integers, like the
reference's; `get_tensor_i8` is the cheaper int8 view of the same data.
"""
import ctypes as C
import os

import numpy as np

from . import capi

# operand layout of each op: names of weight roles in operand order after the
# activation inputs; None marks an operand the INT8 path leaves empty
_WEIGHT_OPERANDS = {
    "tpu.conv_2d": ["filter", "bias", None, None, "rshift", "multiplier"],
    "tpu.deconv_2d": ["filter", "bias", None, None, "rshift", "multiplier"],
    "tpu.fully_connected": ["filter", "bias", None, None, "rshift", "multiplier"],
    "tpu.eltwise_add": [None, None, "rshift", "multiplier"],
    "tpu.eltwise_max": [None, None, "rshift", "multiplier"],
    "tpu.eltwise_min": [None, None, "rshift", "multiplier"],
    "tpu.eltwise_mul": [None, None, "rshift", "multiplier"],
    "tpu.broadcast_add": [None, None, "rshift", "multiplier"],
    "tpu.broadcast_mul": [None, None, "rshift", "multiplier"],
    "tpu.broadcast_sub": [None, None, "rshift", "multiplier"],
    "tpu.pool_avg_2d": [None, None, "rshift", "multiplier"],
    "tpu.pool_max_2d": [],
    "tpu.leaky_relu": [None, None, None, None, "rshift_pos", "multiplier_pos", "rshift_neg",
                       "multiplier_neg"],
    "tpu.prelu": ["slope", None, None, None, None, "rshift_pos", "multiplier_pos", "rshift_neg"],
    "tpu.clip": [None, None, "rshift", "multiplier"],
    "tpu.lut": ["table", None],
    "tpu.scale_lut": ["table"],
    "tpu.relu": [],
    "tpu.quant": [],
    "tpu.pad": [], "tpu.crop": [], "tpu.permute": [], "tpu.reorg": [], "tpu.tile": [],
    "tpu.reverse": [], "tpu.shuffle_channel": [], "tpu.pixelshuffle": [], "tpu.swap_channel": [],
    "tpu.dilate": [], "tpu.reflection_pad": [None, None],
    "tpu.zero_mask": [], "tpu.mul_const": [None, None, None, None],
    "tpu.lrn": ["sqr_lut", "power_lut", None],
    "tpu.reduce_mean": [None, None, "rshift", "multiplier"], "tpu.reduce_sum": [None, None, "rshift", "multiplier"],
    "tpu.reduce_max": [None, None, "rshift", "multiplier"], "tpu.reduce_min": [None, None, "rshift", "multiplier"],
    "tpu.upsample": [],
    "tpu.concat": [None, None, "rshift", "multiplier"],
    "tpu.reshape": [],
    "tpu.input": [],
}


class module:
    version = "tpuhip"

    def __init__(self, device=0, max_batch=1):
        self.lib = capi.bind()
        h = C.c_void_p()
        capi.check(self.lib, self.lib.tpuhip_module_create(device, max_batch, C.byref(h)))
        self.h = h
        self.op_info = []
        self.graph = None
        self._mlir_path = None

    def close(self):
        if self.h:
            self.lib.tpuhip_module_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _ck(self, status):
        capi.check(self.lib, status)

    # -- loading ----------------------------------------------------------
    def load(self, graph, target_op=""):
        """updateWeightMap + loadModule (pymlir.cpp:99-122) for a TPU-dialect .mlir file given by
        name, like pymlir, or for a graph object built in Python."""
        if isinstance(graph, (str, os.PathLike)):
            self.graph = None
            self._mlir_path = os.fspath(graph)
            self._ck(self.lib.tpuhip_module_load_mlir(self.h, os.fspath(graph).encode(),
                                                      target_op.encode() if target_op else None))
            self.op_info = []
            n, t, q = C.c_char_p(), C.c_char_p(), C.c_char_p()
            for i in range(self.lib.tpuhip_module_num_ops(self.h)):
                self._ck(self.lib.tpuhip_module_op_info(self.h, i, C.byref(n), C.byref(t), C.byref(q)))
                self.op_info.append({"name": n.value.decode(), "type": t.value.decode(),
                                     "quant": q.value.decode()})
            return
        self.graph = graph
        self._mlir_path = None
        self._ck(self.lib.tpuhip_module_clear_ops(self.h))
        self.op_info = []
        for op in graph.ops:
            roles = _WEIGHT_OPERANDS.get(op.type)
            if roles is None:
                roles = _WEIGHT_OPERANDS["tpu.lut"] if "table" in op.weights else []
            operands = [s.encode() for s in op.inputs]
            for role in roles:
                if role is None or role not in op.weights:
                    operands.append(b"")
                    continue
                wname = ("%s_%s" % (op.name, role)).encode()
                arr = np.ascontiguousarray(op.weights[role], dtype=np.float32)
                self._ck(self.lib.tpuhip_module_set_weight(self.h, wname, arr.ctypes.data,
                                                           arr.size))
                operands.append(wname)
            shape = (C.c_int64 * len(op.shape))(*op.shape)
            opd = (C.c_char_p * max(len(operands), 1))(*operands)
            keys = [k.encode() for k in op.attrs]
            vals = [float(v) for v in op.attrs.values()]
            ak = (C.c_char_p * max(len(keys), 1))(*keys)
            av = (C.c_double * max(len(vals), 1))(*vals)
            d = capi.OpDescC(op.type.encode(), op.name.encode(), op.quant.encode(),
                             op.param_type.encode(), len(op.shape), shape, len(operands), opd,
                             len(keys), ak, av)
            self._ck(self.lib.tpuhip_module_add_op(self.h, C.byref(d)))
            self.op_info.append({"name": op.name, "type": op.type, "quant": op.quant})
        rets = [s.encode() for s in graph.outputs]
        ra = (C.c_char_p * max(len(rets), 1))(*rets)
        self._ck(self.lib.tpuhip_module_set_returns(self.h, ra, len(rets)))
        self._ck(self.lib.tpuhip_module_load(self.h, target_op.encode() if target_op else None))

    def dump(self):
        """pymlir's module.dump(): the loaded module as text on stderr -- the file's own text when it
        was loaded from a file, else one line per op of the Python-built graph"""
        import sys
        if self._mlir_path:
            sys.stderr.write(open(self._mlir_path).read())
        elif self.graph is not None:
            for op in self.graph.ops:
                sys.stderr.write("%s %s %s %s %s <- %s\n" % (op.type, op.name, op.quant, op.param_type,
                                                              list(op.shape), ", ".join(op.inputs)))

    def set_plugin(self, path):
        """pymlir's module.set_plugin(): custom-op plugins are not part of this build"""
        raise NotImplementedError("custom op plugins are not supported")

    def get_weight_file_path(self):
        return (self.lib.tpuhip_module_weight_file(self.h) or b"").decode()

    def interpret_files(self, mlir_path, tensor_in, tensor_out=None, dump_all_tensor=None):
        """the tpuc-interpreter tool: <mlir> --tensor-in <npz> [--tensor-out <npz>]
        [--dump-all-tensor <npz>]"""
        enc = lambda p: os.fspath(p).encode() if p else None
        self._ck(self.lib.tpuhip_module_interpret_files(self.h, enc(mlir_path), enc(tensor_in),
                                                        enc(tensor_out), enc(dump_all_tensor)))

    def set_option(self, key, value):
        """Options read at the next load(): "fuse_eltwise", "keep_all_tensors" (both default 1)."""
        self._ck(self.lib.tpuhip_module_set_option(self.h, key.encode(), int(value)))

    # -- details ------------------------------------------------------------
    def get_input_details(self):
        out = {}
        for i in range(self.lib.tpuhip_module_num_inputs(self.h)):
            name = self.lib.tpuhip_module_input_name(self.h, i).decode()
            out[name] = int(np.prod(self.tensor_shape(name)))
        return out

    def get_output_details(self):
        return [self.lib.tpuhip_module_output_name(self.h, i).decode()
                for i in range(self.lib.tpuhip_module_num_outputs(self.h))]

    def tensor_names(self):
        return [self.lib.tpuhip_module_tensor_name(self.h, i).decode()
                for i in range(self.lib.tpuhip_module_num_tensors(self.h))]

    def tensor_shape(self, name):
        dims = (C.c_int64 * 8)()
        nd = C.c_int()
        self._ck(self.lib.tpuhip_module_tensor_shape(self.h, name.encode(), dims, C.byref(nd)))
        return tuple(dims[i] for i in range(nd.value))

    def tensor_dtype(self, name):
        r = self.lib.tpuhip_module_tensor_dtype(self.h, name.encode())
        if r is None:
            raise capi.TpuHipError(1, self.lib.tpuhip_last_error().decode())
        return r.decode()

    def kernels(self):
        """(name, algo) of every kernel in execution order"""
        return [(self.lib.tpuhip_module_kernel_name(self.h, i).decode(),
                 self.lib.tpuhip_module_kernel_algo(self.h, i).decode())
                for i in range(self.lib.tpuhip_module_num_kernels(self.h))]

    # -- data ---------------------------------------------------------------
    def set_tensor(self, name, data, bidx=0):
        arr = np.ascontiguousarray(data, dtype=np.float32)
        self._ck(self.lib.tpuhip_module_set_tensor(self.h, name.encode(), arr.ctypes.data,
                                                   arr.size, bidx))

    def set_tensor_i8(self, name, data, bidx=0):
        """int8 NCHW data straight in (no float detour); not for fp32 graph inputs"""
        arr = np.ascontiguousarray(data)
        if arr.dtype != np.int8:
            raise TypeError("set_tensor_i8 takes int8 data, got %s" % arr.dtype)
        self._ck(self.lib.tpuhip_module_set_tensor_i8(self.h, name.encode(), arr.ctypes.data,
                                                      arr.size, bidx))

    def get_tensor(self, name, bidx=0):
        shape = self.tensor_shape(name)
        out = np.empty(shape, np.float32)
        self._ck(self.lib.tpuhip_module_get_tensor(self.h, name.encode(), out.ctypes.data,
                                                   out.size, bidx))
        return out

    def get_tensor_i8(self, name, bidx=0):
        shape = self.tensor_shape(name)
        out = np.empty(shape, np.int8)
        self._ck(self.lib.tpuhip_module_get_tensor_i8(self.h, name.encode(), out.ctypes.data,
                                                      out.size, bidx))
        return out

    def get_all_tensor(self):
        return {n: self.get_tensor(n) for n in self.tensor_names()}

    # -- execution ------------------------------------------------------------
    def invoke(self, bidx=0):
        self._ck(self.lib.tpuhip_module_invoke(self.h, bidx))

    def invoke_to(self, name, bidx=0):
        self._ck(self.lib.tpuhip_module_invoke_to(self.h, name.encode(), bidx))

    def fast_invoke_all_batch(self, name, batch):
        self._ck(self.lib.tpuhip_module_fast_invoke_all_batch(self.h, name.encode(), batch))

    def sync(self):
        self._ck(self.lib.tpuhip_module_sync(self.h))

    def run(self, array, target_op=""):
        """pymlir.module.run (pymlir.cpp:215-269): slice one flat float array over the
        inputs, invoke, return {name: array} for the outputs (or for target_op)."""
        flat = np.ascontiguousarray(array, dtype=np.float32).reshape(-1)
        details = self.get_input_details()
        need = sum(details.values())
        if flat.size != need:
            raise ValueError("input data size %d not same with all input needed size %d" %
                             (flat.size, need))
        off = 0
        for name, size in details.items():
            self.set_tensor(name, flat[off:off + size])
            off += size
        if target_op:
            self.invoke_to(target_op)
            return {target_op: self.get_tensor(target_op)}
        self.invoke()
        return {n: self.get_tensor(n) for n in self.get_output_details()}

    def time_kernels(self, iters=5, bidx=0):
        n = self.lib.tpuhip_module_num_kernels(self.h)
        ms = (C.c_float * max(n, 1))()
        self._ck(self.lib.tpuhip_module_time_kernels(self.h, bidx, iters, ms, n))
        return [(k[0], k[1], ms[i]) for i, k in enumerate(self.kernels())]

    def context_handle(self):
        return self.lib.tpuhip_module_ctx(self.h)
