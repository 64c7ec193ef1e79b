"""Host-side file handling, no GPU: the .npz container (TensorFile) against numpy's own reader
and writer, and the TPU-dialect text reader against hand-written and emitted files."""
import os

import numpy as np
import pytest

from tpu_compiler_amd import capi, graphs, mlir_text

REF_TESTS = "/root/reference/lib/Dialect/TPU/Backend/test"
HERE = os.path.dirname(os.path.abspath(__file__))


def test_npz_written_by_numpy_reads_back(tmp_path):
    rng = np.random.default_rng(1)
    arrays = {"data": rng.normal(size=(2, 3, 5, 7)).astype(np.float32),
              "conv1_filter": rng.integers(-127, 128, (8, 3, 3, 3)).astype(np.float32),
              "scalar": np.float32(2.5), "empty": np.zeros((0, 4), np.float32),
              "vec": np.arange(1000, dtype=np.float32)}
    for saver, name in ((np.savez, "plain.npz"), (np.savez_compressed, "deflated.npz")):
        path = tmp_path / name
        saver(path, **arrays)
        f = capi.TensorFile(path)
        assert sorted(f.names()) == sorted(arrays)
        for k, v in arrays.items():
            shape, kind, ws = f.info(k)
            assert shape == np.shape(v) and kind == "f" and ws == 4
            assert np.array_equal(f.read(k), v)
        f.close()


def test_npz_written_here_is_read_by_numpy(tmp_path):
    rng = np.random.default_rng(2)
    path = tmp_path / "out.npz"
    f = capi.TensorFile(path, "w")
    arrays = {"fc": rng.normal(size=(32, 1000)).astype(np.float32),
              "x": rng.normal(size=(1, 3, 4, 5)).astype(np.float32),
              "one": np.array([7.0], np.float32), "zero_d": np.float32(-1.5).reshape(())}
    for k, v in arrays.items():
        f.add(k, v)
    with pytest.raises(capi.TpuHipError, match="already exist"):
        f.add("fc", arrays["fc"])
    f.keep()
    f.close()
    with np.load(path) as z:
        assert sorted(z.files) == sorted(arrays)
        for k, v in arrays.items():
            assert z[k].dtype == np.float32 and z[k].shape == v.shape and np.array_equal(z[k], v)
    # append mode keeps what is there; delete removes; keep rewrites the whole file
    f = capi.TensorFile(path, "a")
    f.delete("one")
    f.add("extra", np.ones((2, 2), np.float32))
    with pytest.raises(capi.TpuHipError, match="to delete"):
        f.delete("nope")
    f.keep()
    f.close()
    with np.load(path) as z:
        assert sorted(z.files) == ["extra", "fc", "x", "zero_d"]
        assert np.array_equal(z["fc"], arrays["fc"])


def test_npz_errors_like_the_reference(tmp_path):
    with pytest.raises(capi.TpuHipError, match="doesn't exist"):
        capi.TensorFile(tmp_path / "missing.npz")
    bad = tmp_path / "bad.npz"
    bad.write_bytes(b"this is not a zip archive at all, just text long enough")
    with pytest.raises(capi.TpuHipError, match="not a zip"):
        capi.TensorFile(bad)
    path = tmp_path / "ints.npz"
    np.savez(path, w=np.arange(6, dtype=np.int8).reshape(2, 3), f=np.zeros(3, np.float32))
    f = capi.TensorFile(path)
    assert f.info("w") == ((2, 3), "i", 1)
    with pytest.raises(capi.TpuHipError, match="size does not match"):   # readTensor<float> is float32 only
        f.read("w")
    with pytest.raises(capi.TpuHipError, match="failed to find tensor"):
        f.read("absent")
    out = np.empty(5, np.float32)
    with pytest.raises(capi.TpuHipError, match="size does not match"):
        capi.check(f.lib, f.lib.tpuhip_npz_read_f32(f.h, b"f", out.ctypes.data, 5))
    f.close()


HAND_WRITTEN = r'''
// a quantized conv + relu6 clip, written by hand in the syntax of the reference's op tests
module attributes {tpu.dummy = 1 : i32} {
  func @tpu_func(%arg0: tensor<1x3x8x8xsi8>) -> (tensor<1x4x4x4xsi8>, tensor<1x4x4x4xsi8>) attributes {chipname = "cv183x"} {
    %0 = "tpu.weight_file"() {filename = "w_1_06eeeb7e.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "INT8", param_type = "NONE", threshold = 2.640000e+00 : f32}} : (tensor<1x3x8x8xsi8>) -> tensor<1x3x8x8xsi8> loc("data")
    %2 = "tpu.load_weight"(%0) {name = "conv_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<4x3x3x3xf32>
    %3 = "tpu.load_weight"(%0) {name = "conv_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<4xf32>
    %4 = "tpu.none"() : () -> none
    %5 = "tpu.load_weight"(%0) {name = "conv_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<4xf32>
    %6 = "tpu.load_weight"(%0) {name = "conv_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<4xf32>
    %7 = "tpu.conv_2d"(%1, %2, %3, %4, %4, %5, %6) {do_relu = true, name = "conv", param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0x40A8F5C3 : f32}} : (tensor<1x3x8x8xsi8>, tensor<4x3x3x3xf32>, tensor<4xf32>, none, none, tensor<4xf32>, tensor<4xf32>) -> tensor<1x4x4x4xsi8>
    %8 = "tpu.pad"(%7) {const_val = 0.000000e+00 : f32, mode = "edge", name = "pad", pads = [0 : i32, 0 : i32, 1 : i32, 1 : i32, 0 : i32, 0 : i32, 1 : i32, 1 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 1.0 : f32}} : (tensor<1x4x4x4xsi8>) -> tensor<1x4x6x6xsi8>
    %9 = "tpu.crop"(%8) {crop_offset = [0 : i32, 0 : i32, 1 : i32, 1 : i32], name = "crop", quant = {mode = "INT8", param_type = "NONE", threshold = 1.0 : f32}, weird = dense<[1, 2]> : tensor<2xi32>, unit_flag} : (tensor<1x4x6x6xsi8>) -> tensor<1x4x4x4xsi8>
    return %7, %9 : tensor<1x4x4x4xsi8>, tensor<1x4x4x4xsi8>
  }
}
'''


def _describe(tmp_path, text, name="m.mlir"):
    p = tmp_path / name
    p.write_text(text)
    return capi.mlir_describe(p)


def test_reader_understands_a_hand_written_quantized_module(tmp_path):
    d = _describe(tmp_path, HAND_WRITTEN).splitlines()
    assert d[0] == "weight_file w_1_06eeeb7e.npz" and d[1] == "chipname cv183x"
    assert "weight conv_filter INT8 [4,3,3,3]" in d and "weight conv_multiplier UINT32 [4]" in d
    ops = [l for l in d if l.startswith("op ")]
    assert ops[0].startswith("op tpu.input data INT8 NONE [1,3,8,8] {")
    conv = ops[1]
    assert conv.startswith("op tpu.conv_2d conv INT8 RSHIFT_AND_M_I32 [1,4,4,4] data conv_filter conv_bias - - "
                           "conv_rshift conv_multiplier {")
    for frag in ("do_relu=1", "kernel_h=3", "stride_w=2", "padding_t=1", "with_bias=1", "is_dw=0", "group=1",
                 "ins_h=0", "ins_w=0", "padding_same=1"):
        assert frag in conv, frag
    thr = float(conv.split("threshold=")[1].split(",")[0].rstrip("}"))
    assert abs(thr - np.frombuffer(np.uint32(0x40A8F5C3).tobytes(), np.float32)[0]) < 1e-4   # bit-pattern float
    assert "mode_edge=1" in ops[2] and "pads2=1" in ops[2] and "pads7=1" in ops[2] and "pads0=0" in ops[2]
    assert "crop_offset3=1" in ops[3] and "unit_flag=1" in ops[3] and "weird" not in ops[3]
    assert d[-2:] == ["return conv", "return crop"]


@pytest.mark.parametrize("text, message", [
    ("module {\n}\n", "mlir:2: unexpected '}' at top level"),
    ("// nothing here\n", "no func found"),
    ('func @f() {\n  %0 = "tpu.none"() : () -> none\n', "func body not closed"),
    ('func @f(%arg0: tensor<1xf32>) -> tensor<1xf32> {\n  %0 = tpu.relu %arg0 : tensor<1xf32>\n}', "mlir:2: .*generic form"),
    ('func @f(%arg0: tensor<1xf32>) -> tensor<1xf32> {\n  %0 = "tpu.relu"(%9) {name = "r"} : (tensor<1xf32>) -> tensor<1xf32>\n  return %0 : tensor<1xf32>\n}',
     "mlir:2: .*undefined value %9"),
    ('func @f(%arg0: tensor<1xf32>) -> tensor<1xf32> {\n  %0 = "tpu.relu"(%arg0) : (tensor<1xf32>) -> tensor<1xf32>\n}', "no name attribute"),
    ('func @f(%arg0: tensor<?x3xf32>) -> tensor<?x3xf32> {\n  %0 = "tpu.relu"(%arg0) {name = "r"} : (tensor<?x3xf32>) -> tensor<?x3xf32>\n}', "dynamic shapes"),
    ('func @f(%arg0: tensor<1xf32>) -> tensor<1xf32> {\n  %0 = "tpu.relu"(%arg0, %arg0) {name = "r"} : (tensor<1xf32>) -> tensor<1xf32>\n}',
     "2 operands but 1 operand types"),
    ('func @f() {\n  %0 = "tpu.x"() {name = "unterminated} : () -> none\n}', "unterminated string"),
])
def test_reader_reports_malformed_text_with_its_line(tmp_path, text, message):
    with pytest.raises(capi.TpuHipError, match=message):
        _describe(tmp_path, text)
    with pytest.raises(capi.TpuHipError, match="cannot open"):
        capi.mlir_describe(tmp_path / "absent.mlir")


@pytest.mark.skipif(not os.path.isdir(REF_TESTS), reason="the reference checkout is not on this machine")
def test_reader_accepts_the_references_own_op_test_graphs():
    """every single-function .mlir the reference's backend tests hold parses, and the facts that
    can be read off the text by eye come out: op types in order, names, shapes, operand wiring"""
    seen = 0
    for fn in sorted(os.listdir(REF_TESTS)):
        if not fn.endswith(".mlir"):
            continue
        text = capi.mlir_describe(os.path.join(REF_TESTS, fn))
        assert text.startswith("weight_file ") and "\nreturn " in text, fn
        seen += 1
    assert seen >= 30
    d = capi.mlir_describe(os.path.join(REF_TESTS, "conv.mlir")).splitlines()
    assert d[0] == "weight_file conv_06eeeb7e.npz"
    assert "weight filter NONE [32,3,3,3]" in d and "weight bias NONE [32]" in d
    conv = [l for l in d if l.startswith("op tpu.conv_2d")][0]
    assert conv.startswith("op tpu.conv_2d conv NONE NONE [4,32,112,112] data filter bias - - - - {")
    for frag in ("stride_h=2", "padding_b=1", "do_relu=0", "with_bias=1", "kernel_h=3", "kernel_w=3"):
        assert frag in conv, frag      # kernel size from the filter type: this file predates kernel_h
    assert d[-1] == "return conv"
    d = capi.mlir_describe(os.path.join(REF_TESTS, "eltwise_add.mlir"))
    assert "op tpu.eltwise_add " in d


@pytest.mark.skipif(not os.path.isdir(REF_TESTS), reason="the reference checkout is not on this machine")
def test_reader_output_equals_descriptions_typed_in_by_hand():
    """the reader against an independent statement of what five of the reference's op-test graphs say
    (tests/golden/reference_graph_facts.json, typed from the files' text): weight file, weights with
    their shapes, every op in order with type / name / quant mode / param type / shape / operand wiring
    (none operands included), every attribute value the file writes, the returned values in order"""
    import json
    facts = json.load(open(os.path.join(HERE, "golden", "reference_graph_facts.json")))
    for name, want in facts.items():
        if name.startswith("_"):
            continue
        d = capi.mlir_describe(os.path.join(REF_TESTS, name + ".mlir")).splitlines()
        assert d[0] == "weight_file " + want["weight_file"], name
        weights = [l.split(" ") for l in d if l.startswith("weight ")]
        assert [(w[1], w[2], w[3]) for w in weights] == \
            [(n, "NONE", "[" + ",".join(map(str, shp)) + "]") for n, shp in want["weights"]], name
        ops = [l for l in d if l.startswith("op ")]
        assert len(ops) == len(want["ops"]), name
        for line, op in zip(ops, want["ops"]):
            head, attrs = line.split(" {")
            f = head.split()
            assert f[1:5] == [op["type"], op["name"], op["quant"], op["param_type"]], line
            assert f[5] == "[" + ",".join(map(str, op["shape"])) + "]", line
            assert f[6:] == op["operands"], line
            got = dict(kv.split("=") for kv in attrs.rstrip("}").split(",") if kv)
            for k, v in op["attrs"].items():
                assert k in got and float(got[k]) == float(v), (name, op["name"], k, got.get(k))
        assert [l.split()[1] for l in d if l.startswith("return ")] == want["returns"], name


def test_emitted_text_reads_back_as_the_same_graph(tmp_path):
    """graph -> .mlir + .npz -> reader: every op with its type, name, quant mode, shape, operand
    wiring (weights by name, absent operands as none) and every attribute value"""
    g = graphs.CONFIGS["cfg2"](batch=2)
    path = tmp_path / "cfg2.mlir"
    wfile = mlir_text.write_mlir(g, path)
    d = capi.mlir_describe(path).splitlines()
    assert d[0] == "weight_file " + os.path.basename(wfile)
    ops = [l for l in d if l.startswith("op ")]
    assert len(ops) == len(g.ops)
    from tpu_compiler_amd.pymodule import _WEIGHT_OPERANDS
    for line, op in zip(ops, g.ops):
        head, attrs = line.split(" {")
        f = head.split()
        assert f[1:5] == [op.type, op.name, op.quant, op.param_type], line
        assert f[5] == "[" + ",".join(str(v) for v in op.shape) + "]"
        want = list(op.inputs) if op.type != "tpu.input" else []
        for role in _WEIGHT_OPERANDS.get(op.type, []):
            want.append("%s_%s" % (op.name, role) if role and role in op.weights else "-")
        assert f[6:] == want, line
        got = dict(kv.split("=") for kv in attrs.rstrip("}").split(",") if kv)
        for k, v in op.attrs.items():
            assert float(got[k]) == float(v), (op.name, k)
    assert [l.split()[1] for l in d if l.startswith("return ")] == list(g.outputs)
    with np.load(wfile) as z:
        for op in g.ops:
            for role, arr in op.weights.items():
                key = "%s_%s" % (op.name, role)
                if key in z.files:
                    assert z[key].dtype == np.float32 and np.array_equal(z[key], arr.astype(np.float32))


def test_damaged_files_raise_errors_and_never_crash(tmp_path):
    """truncated and bit-flipped archives / texts either load or are refused with an error"""
    rng = np.random.default_rng(11)
    good = tmp_path / "good.npz"
    np.savez(good, a=np.arange(40, dtype=np.float32).reshape(5, 8), b=np.ones((3, 3), np.float32))
    blob = good.read_bytes()
    outcomes = {"ok": 0, "refused": 0}
    for trial in range(300):
        data = bytearray(blob)
        if trial % 3 == 0:
            data = data[:int(rng.integers(0, len(data)))]
        else:
            for _ in range(int(rng.integers(1, 4))):
                data[int(rng.integers(0, len(data)))] = int(rng.integers(0, 256))
        p = tmp_path / "damaged.npz"
        p.write_bytes(bytes(data))
        try:
            f = capi.TensorFile(p)
            for name in f.names():
                try:
                    f.read(name)
                except capi.TpuHipError:
                    pass
            f.close()
            outcomes["ok"] += 1
        except capi.TpuHipError:
            outcomes["refused"] += 1
    assert outcomes["refused"] > 50 and outcomes["ok"] > 10
    # crafted zip64 records whose 64-bit offsets sit just under 2^64: offset + record size wraps, so
    # only a check against the bytes that are left refuses them
    import struct
    eocd = blob.rfind(b"PK\x05\x06")
    cd_off = struct.unpack_from("<I", blob, eocd + 16)[0]
    for e64_off, cd64, lho64 in ((2**64 - 8, cd_off, None), (None, 2**64 - 40, None), (None, cd_off, 2**64 - 29)):
        body = bytearray(blob[:eocd])
        if lho64 is not None:
            # first central entry: local header offset escapes to a zip64 extra field
            struct.pack_into("<I", body, cd_off + 42, 0xffffffff)
            nlen, xlen = struct.unpack_from("<HH", body, cd_off + 28)
            extra = struct.pack("<HHQ", 1, 8, lho64)
            struct.pack_into("<H", body, cd_off + 30, xlen + len(extra))
            at = cd_off + 46 + nlen + xlen
            body[at:at] = extra
        rec64_at = len(body)
        rec64 = struct.pack("<IQHHIIQQQQ", 0x06064b50, 44, 45, 45, 0, 0, 2, 2, len(body) - cd_off, cd64)
        loc64 = struct.pack("<IIQI", 0x07064b50, 0, rec64_at if e64_off is None else e64_off, 1)
        tail = bytearray(blob[eocd:eocd + 22])
        struct.pack_into("<HH", tail, 8, 0xffff, 0xffff)
        struct.pack_into("<I", tail, 16, 0xffffffff)
        p = tmp_path / "zip64.npz"
        p.write_bytes(bytes(body) + rec64 + loc64 + bytes(tail))
        with pytest.raises(capi.TpuHipError):
            capi.TensorFile(p)
    text = HAND_WRITTEN
    refused = 0
    for trial in range(200):
        cut = int(rng.integers(0, len(text)))
        t = text[:cut] if trial % 2 == 0 else text[:cut] + "@#}{" + text[cut + 3:]
        try:
            _describe(tmp_path, t, "damaged.mlir")
        except capi.TpuHipError:
            refused += 1
    assert refused > 150
