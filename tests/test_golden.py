"""The committed vectors under tests/golden/: small quantized graphs as TPU-dialect text +
weight file, with every tensor of each graph as the oracle computed it when the fixtures
were written (tests/golden/make_fixtures.py).

CPU: the oracle of this tree still reproduces every stored tensor, the stored graph text
still parses to the graph the generator builds, and the vectors are not degenerate.
GPU: the HIP path loads the stored files through the C ABI and must produce the stored
tensors bit for bit -- nothing on that side is computed by the oracle at test time."""
import importlib.util
import os

import numpy as np
import pytest

from tpu_compiler_amd import capi, module

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
fixtures = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(fixtures)

NAMES = [fn.__name__ for fn in fixtures.GRAPHS]


def described(name):
    """weight file, [(type, name, shape)] and returned names, from the reader's own account of
    the stored text"""
    weight_file, ops, returns = None, [], []
    for line in capi.mlir_describe(os.path.join(GOLDEN, name + ".mlir")).splitlines():
        f = line.split(" ")
        if f[0] == "weight_file":
            weight_file = f[1]
        elif f[0] == "op":
            shape = next(t for t in f[3:] if t.startswith("["))
            ops.append((f[1], f[2], tuple(int(v) for v in shape[1:-1].split(","))))
        elif f[0] == "return":
            returns.append(f[1])
    return weight_file, ops, returns


def stored(name):
    with np.load(os.path.join(GOLDEN, name + "_io.npz")) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("fn", fixtures.GRAPHS, ids=NAMES)
def test_oracle_reproduces_the_stored_tensors(fn):
    g, x = fixtures.build(fn)
    want = fixtures.expected(g, x)
    have = stored(g.name)
    assert sorted(have) == sorted(want)
    for op in g.ops:
        assert have[op.name].dtype == want[op.name].dtype, op.name
        assert np.array_equal(have[op.name], want[op.name]), op.name
    assert np.array_equal(have[g.input_op().name], x)


@pytest.mark.parametrize("name", NAMES)
def test_stored_vectors_are_not_degenerate(name):
    """a fixture whose tensors were all zero or all saturated would pin nothing"""
    for key, v in stored(name).items():
        if v.size < 64:
            continue
        assert len(np.unique(v)) > 8, key
        if v.dtype == np.int8:
            assert np.mean((v == 127) | (v == -128)) < 0.5, key


@pytest.mark.parametrize("fn", fixtures.GRAPHS, ids=NAMES)
def test_stored_graph_text_describes_the_generated_graph(fn):
    g, _ = fixtures.build(fn)
    weight_file, ops, returns = described(g.name)
    assert weight_file == g.name + "_weights.npz"
    assert ops == [(o.type, o.name, tuple(o.shape)) for o in g.ops]
    assert returns == list(g.outputs)
    with np.load(os.path.join(GOLDEN, g.name + "_weights.npz")) as z:
        for op in g.ops:
            for role, arr in op.weights.items():
                assert np.array_equal(z["%s_%s" % (op.name, role)].ravel(),
                                      np.asarray(arr, np.float32).ravel()), (op.name, role)


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("fused", [1, 0])
def test_hip_path_reproduces_the_stored_tensors(name, fused):
    have = stored(name)
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.set_option("fuse_eltwise", fused)
    m.load(os.path.join(GOLDEN, name + ".mlir"))
    info = {i["name"]: i for i in m.op_info}
    assert sorted(info) == sorted(have)
    inp = m.op_info[0]["name"]
    m.set_tensor(inp, have[inp].astype(np.float32))
    m.invoke()
    for key, want in have.items():
        if want.dtype == np.int8:
            got = m.get_tensor_i8(key)
        else:
            got = m.get_tensor(key)
        assert got.shape == want.shape, key
        assert np.array_equal(got, want.astype(got.dtype)), key
    m.close()


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_file_to_file_run_reproduces_the_stored_outputs(name, tmp_path):
    """the way the tpuc-interpreter tool is used: graph file + input .npz -> output .npz"""
    have = stored(name)
    _, ops, returns = described(name)
    inp = ops[0][1]
    np.savez(tmp_path / "in.npz", **{inp: have[inp].astype(np.float32)})
    m = module()
    m.interpret_files(os.path.join(GOLDEN, name + ".mlir"), tmp_path / "in.npz", tmp_path / "out.npz")
    m.close()
    with np.load(tmp_path / "out.npz") as z:
        assert sorted(z.files) == sorted(returns)
        for key in z.files:
            assert np.array_equal(z[key], have[key].astype(np.float32)), key
