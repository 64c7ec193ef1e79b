"""The reference's own op-test graphs (lib/Dialect/TPU/Backend/test/*.mlir), quantized by this
repository's pass with seeded pseudo-weights (tests/golden/make_opgraph_fixtures.py writes the
quantized text and weights kept under tests/golden/opgraphs/), run end to end.

CPU: the stored files read back and describe INT8 graphs the oracle can run.
GPU: the HIP path loads the stored files through the C ABI; every tensor of every graph --
quantized input, each op's int8 result, dequantized output -- equals the oracle's on a seeded input."""
import importlib.util
import os

import numpy as np
import pytest

import mlir_graph
import oracle_graph
from tpu_compiler_amd import module

HERE = os.path.dirname(os.path.abspath(__file__))
OPGRAPHS = os.path.join(HERE, "golden", "opgraphs")
_spec = importlib.util.spec_from_file_location("make_opgraph_fixtures",
                                               os.path.join(HERE, "golden", "make_opgraph_fixtures.py"))
_fx = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_fx)
NAMES = list(_fx.GRAPHS)


def _inputs(g, seed):
    """fp32 inputs spread over a little more than the range their thresholds cover"""
    rng = np.random.default_rng(seed)
    out = {}
    for op in g.ops:
        if op.type == "tpu.input":
            thr = float(op.attrs.get("threshold", 1.0))
            out[op.name] = (rng.normal(0, 0.45 * thr, op.shape)).astype(np.float32)
    return out


@pytest.mark.parametrize("name", NAMES)
def test_stored_op_graphs_are_int8_graphs_the_oracle_covers(name, tmp_path):
    g = mlir_graph.load(_fx.materialize(name, tmp_path))
    body = [op for op in g.ops if op.type not in ("tpu.input", "tpu.quant", "tpu.reshape")]
    assert body and all(op.quant in ("INT8", "UINT8") for op in body), [(o.name, o.quant) for o in body]
    assert g.outputs and all(g.by_name[o].type == "tpu.quant" for o in g.outputs)
    for op in g.ops:
        for role, arr in op.weights.items():
            assert np.array_equal(arr, np.rint(arr)) or role in ("slope",), (op.name, role)


@pytest.mark.parametrize("name", ["fc", "tile", "avg_pool"])
def test_oracle_runs_the_small_stored_op_graphs(name):
    g = mlir_graph.load(os.path.join(OPGRAPHS, name + "_int8.mlir"))
    for k, v in _inputs(g, 5).items():
        g.by_name[k].data = v
    out = oracle_graph.run(g)
    for op in g.ops:
        assert out[op.name].shape == tuple(op.shape), op.name
    mid = next(op for op in g.ops if op.type not in ("tpu.input", "tpu.quant", "tpu.reshape"))
    assert len(np.unique(out[mid.name])) > 8


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_hip_path_runs_the_reference_op_graphs_like_the_oracle(name, tmp_path):
    path = _fx.materialize(name, tmp_path)
    g = mlir_graph.load(path)
    xs = _inputs(g, 11 + len(name))
    for k, v in xs.items():
        g.by_name[k].data = v
    want = oracle_graph.run(g)
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.load(path)
    for k, v in xs.items():
        m.set_tensor(k, v)
    m.invoke()
    checked = 0
    for op in g.ops:
        if op.type == "tpu.input":
            continue
        w = want[op.name]
        got = m.get_tensor(op.name) if w.dtype == np.float32 else m.get_tensor_i8(op.name)
        assert np.array_equal(np.asarray(got).reshape(w.shape), w), (name, op.name, op.type)
        checked += 1
    assert checked >= 2
    m.close()
