"""The C++ op-level API (the reference's class names and operand conventions) driven from a plain
C++ program, tests/cpp/op_kernels_example.cpp, built by __graft_entry__.build().  The program
writes its operands and every result tensor to an .npz through the C++ TensorFile; here they are
checked against the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "op_kernels_example.bin")


def test_cpp_op_kernels_match_the_oracle(tmp_path):
    assert os.path.exists(BIN), "build it with __graft_entry__.build()"
    out = tmp_path / "tensors.npz"
    res = subprocess.run([BIN, str(out)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    lines = res.stdout.splitlines()
    assert lines[0].split()[:3] == ["data", "tpu.input", "INT8"] and lines[1].split()[1] == "tpu.conv_2d"
    z = np.load(out)
    x = z["data"].astype(np.int8)
    assert z["data"].dtype == np.float32 and x.shape == (2, 24, 12, 12)

    def conv(name, src, k, pad, relu):
        w = z[name + "_filter"].astype(np.int8)
        d = O.make_conv_desc(src.shape, w.shape, 1, (1, 1), (pad,) * 4, (1, 1), (0, 0), relu, True, None)
        return O.conv2d_i8(src, w, z[name + "_bias"], z[name + "_rshift"], z[name + "_multiplier"], d)

    c1 = conv("conv1", x, 3, 1, True)
    c2 = conv("conv2", c1, 1, 0, False)
    add = O.eltwise_add_i8([c1, c2], z["add_multiplier"], z["add_rshift"], True)
    gap = O.pool_avg_i8(add, O.make_pool_desc(add.shape, (12, 12), (1, 1), (0, 0, 0, 0)), z["gap_rshift"][0],
                        z["gap_multiplier"][0])
    for name, want in (("conv1", c1), ("conv2", c2), ("add", add), ("gap", gap)):
        assert z[name].shape == want.shape and np.array_equal(z[name], want.astype(np.float32)), name
        assert len(np.unique(want)) > 8
