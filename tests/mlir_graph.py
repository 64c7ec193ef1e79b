"""Test infrastructure: a quantized .mlir file + its weight .npz as a graphs.Graph, so that the
oracle (tests/oracle_graph.py) can run what the HIP path loads from the same files.  The text is
read by the library's own reader (tpuhip_mlir_describe); this module only arranges its account:
which operands are activations, which weights, and under which role the oracle expects each."""
import os

import numpy as np

from tpu_compiler_amd import capi, graphs
from tpu_compiler_amd.pymodule import _WEIGHT_OPERANDS


def _attrs(text):
    out = {}
    body = text.strip()[1:-1]
    for item in body.split(",") if body else []:
        k, v = item.split("=", 1)
        out[k] = float(v)
        if out[k] == int(out[k]) and "." not in v and "e" not in v.lower():
            out[k] = int(out[k])
    return out


def load(mlir_path):
    """-> (Graph, {input name: shape}); ops keep the file's names, quant modes and attributes"""
    desc = capi.mlir_describe(str(mlir_path)).splitlines()
    wfile = next(l.split(" ")[1] for l in desc if l.startswith("weight_file "))
    wpath = os.path.join(os.path.dirname(str(mlir_path)), wfile)
    weights = {}
    if os.path.exists(wpath):
        with np.load(wpath) as z:
            weights = {k: z[k] for k in z.files}
    g = graphs.Graph(os.path.splitext(os.path.basename(str(mlir_path)))[0], 0)
    for line in desc:
        f = line.split(" ")
        if f[0] == "return":
            g.outputs.append(f[1])
        if f[0] != "op":
            continue
        type_, name, quant, ptype = f[1:5]
        shape = tuple(int(v) for v in f[5][1:-1].split(",") if v)
        operands = [t for t in f[6:] if not t.startswith("{")]
        attrs = _attrs(f[-1]) if f[-1].startswith("{") else {}
        inputs = []
        while operands and operands[0] in g.by_name:
            inputs.append(operands.pop(0))
        roles = _WEIGHT_OPERANDS.get(type_)
        assert roles is not None, type_
        wts = {}
        for role, wname in zip(roles, operands):
            if role is not None and wname != "-":
                wts[role] = np.asarray(weights[wname], np.float32)
        op = g.add(graphs.Op(type_, name, inputs, shape, attrs, wts, ptype))
        op.quant = quant
    return g
