"""The calibration-table import + INT8 quantisation pass over TPU-dialect files
(tpuhip_quantize_mlir_files; the reference's tpuc-opt --import-calibration-table --tpu-quant).

CPU: an fp32 network written as text + weights is quantised from files; every tensor of the
weight file it writes must equal what the per-op arithmetic helpers (pinned in
test_quantize.py) give for the same thresholds, the text must say INT8 where it should and
carry tpu.quant ops at the fp32 edges with the reference's names and scales; threshold
propagation rules; refusals; the reference's own fp32 op graphs go through.
GPU: the files the pass wrote run through module.load: bit-exact against the oracle on an
independently built INT8 graph, and close to the fp32 network they came from."""
import os
import re

import numpy as np
import pytest

import oracle_graph
from tpu_compiler_amd import capi, graphs, mlir_text, module
from tpu_compiler_amd import quantize as Q

REF_TESTS = "/root/reference/lib/Dialect/TPU/Backend/test"


def fp32_op(g, type_, name, inputs, shape, attrs=None, weights=None):
    op = graphs.Op(type_, name, inputs, shape, attrs or {}, weights or {})
    op.quant = "NONE"
    g.add(op)
    return name


def conv_attrs(k, pad, relu, stride=1, group=1):
    return dict(kernel_h=k, kernel_w=k, stride_h=stride, stride_w=stride, dilation_h=1, dilation_w=1,
                padding_t=pad, padding_b=pad, padding_l=pad, padding_r=pad, group=group, do_relu=int(relu),
                with_bias=1)


def small_network():
    """-> (fp32 graph, torch activations by op name, input array)"""
    import torch
    import torch.nn.functional as F
    torch.manual_seed(11)
    rng = np.random.default_rng(11)
    n, hw = 2, 12
    x = torch.tensor(rng.normal(0, 1, (n, 8, hw, hw)).astype(np.float32)).clamp(-3, 3)
    w1, b1 = torch.randn(16, 8, 3, 3) * 0.15, torch.randn(16) * 0.2
    w2, b2 = torch.randn(16, 16, 3, 3) * 0.1, torch.randn(16) * 0.2
    w3, b3 = torch.randn(24, 32, 1, 1) * 0.2, torch.randn(24) * 0.1
    wf, bf = torch.randn(10, 24) * 0.4, torch.randn(10) * 0.1
    a1 = F.relu(F.conv2d(x, w1, b1, padding=1))
    a2 = F.conv2d(a1, w2, b2, padding=1)
    a3 = F.relu(a1 + a2)
    p = F.max_pool2d(a3, 2, 2)
    u = F.interpolate(p, scale_factor=2, mode="nearest")
    cat = torch.cat([u, a2], 1)
    a4 = F.conv2d(cat, w3, b3)
    a5 = F.leaky_relu(a4, 0.1)
    sg = torch.sigmoid(a5)
    ml = a5 * sg
    a6 = ml.mean(dim=(2, 3), keepdim=True)
    a7 = F.linear(a6.flatten(1), wf, bf)
    acts = dict(input=x, c1=a1, c2=a2, add=a3, pool=p, up=u, cat=cat, c3=a4, leaky=a5, sig=sg, mul=ml, gap=a6, fc=a7)

    g = graphs.Graph("fp32_net", 0)
    xin = graphs.Op("tpu.input", "input", [], (n, 8, hw, hw))
    xin.quant = "NONE"
    xin.data = x.numpy()
    g.add(xin)
    f = lambda t: t.numpy().astype(np.float32)
    fp32_op(g, "tpu.conv_2d", "c1", ["input"], (n, 16, hw, hw), conv_attrs(3, 1, True), dict(filter=f(w1), bias=f(b1)))
    fp32_op(g, "tpu.conv_2d", "c2", ["c1"], (n, 16, hw, hw), conv_attrs(3, 1, False), dict(filter=f(w2), bias=f(b2)))
    fp32_op(g, "tpu.eltwise_add", "add", ["c1", "c2"], (n, 16, hw, hw), dict(do_relu=1))
    fp32_op(g, "tpu.pool_max_2d", "pool", ["add"], (n, 16, hw // 2, hw // 2),
            dict(kernel_h=2, kernel_w=2, stride_h=2, stride_w=2, padding_t=0, padding_b=0, padding_l=0, padding_r=0,
                 do_relu=0, count_include_pad=0))
    fp32_op(g, "tpu.upsample", "up", ["pool"], (n, 16, hw, hw), dict(scale_h=2, scale_w=2))
    fp32_op(g, "tpu.concat", "cat", ["up", "c2"], (n, 32, hw, hw), dict(axis=1, do_relu=0))
    fp32_op(g, "tpu.conv_2d", "c3", ["cat"], (n, 24, hw, hw), conv_attrs(1, 0, False), dict(filter=f(w3), bias=f(b3)))
    fp32_op(g, "tpu.leaky_relu", "leaky", ["c3"], (n, 24, hw, hw), dict(negative_slope=0.1))
    fp32_op(g, "tpu.sigmoid", "sig", ["leaky"], (n, 24, hw, hw), dict(scale=1.0, bias=0.0))
    fp32_op(g, "tpu.eltwise_mul", "mul", ["leaky", "sig"], (n, 24, hw, hw), dict(do_relu=0))
    fp32_op(g, "tpu.pool_avg_2d", "gap", ["mul"], (n, 24, 1, 1),
            dict(kernel_h=hw, kernel_w=hw, stride_h=1, stride_w=1, padding_t=0, padding_b=0, padding_l=0, padding_r=0,
                 do_relu=0, count_include_pad=0))
    fp32_op(g, "tpu.reshape", "flat", ["gap"], (n, 24))
    fp32_op(g, "tpu.fully_connected", "fc", ["flat"], (n, 10), dict(do_relu=0), dict(filter=f(wf), bias=f(bf)))
    g.outputs = ["fc"]
    return g, acts, x.numpy()


def thresholds_after_import(thr):
    """what the table import turns the measured thresholds into for small_network(): the add's
    single-use consumer chain pool -> up pulls `add` to the concat-side value, etc."""
    t = dict(thr)
    # concat: `up` has one use -> takes cat's; c2 has two uses -> keeps its own
    t["up"] = t["cat"]
    # backward: pool (max pool) sets add (one use) to pool's; leaky sets c3 (one use) to leaky's
    t["add"] = t["pool"]
    t["c3"] = t["leaky"]
    # forward: pool takes add's (equal already), up takes pool's -- overriding the concat step
    t["up"] = t["pool"]
    t["sig"] = 1.0
    return t


def measured_thresholds(acts):
    """max |activation| per op, as the float the table's seven printed digits read back to"""
    return {k: float(np.float32(float("%.7g" % float(v.abs().max())))) for k, v in acts.items()}


def write_inputs(tmp_path, g, thr):
    path = tmp_path / "net_fp32.mlir"
    mlir_text.write_mlir(g, path)
    table = tmp_path / "cali_table"
    with open(table, "w") as f:
        f.write("# genetated time: now\n# op_name    threshold\n")
        for k, v in thr.items():
            f.write("%s %.7g\n" % (k, v) if k != "c2" else "%s %.7g -1.5 2.5\n" % (k, v))
    return path, table


def describe(path):
    ops, weights, returns = {}, {}, []
    for line in capi.mlir_describe(path).splitlines():
        w = line.split(" ")
        if w[0] == "op":
            ops[w[2]] = dict(type=w[1], quant=w[3], param=w[4], line=line)
        elif w[0] == "weight":
            weights[w[1]] = w[2]
        elif w[0] == "return":
            returns.append(w[1])
    return ops, weights, returns


def f32_attr(mlir_path, op_name, key):
    """float attribute `key` of the op named op_name, read from the text at full precision"""
    import struct
    for line in open(mlir_path).read().splitlines():
        if 'name = "%s"' % op_name in line:
            tok = re.search(r"\b%s = ([-+0-9.eExXa-fA-F]+) : f32" % key, line).group(1)
            if tok.lower().startswith("0x"):
                return np.float32(struct.unpack("<f", struct.pack("<I", int(tok, 16)))[0])
            return np.float32(float(tok))
    raise KeyError(op_name)


def expected_int8_graph(g32, thr, x):
    """the INT8 graph the pass should be equivalent to, built op by op from the arithmetic helpers"""
    t = thresholds_after_import(thr)
    n, hw = x.shape[0], x.shape[2]
    g = graphs.Graph("expected", 0)
    fin = graphs.Op("tpu.input", "input", [], x.shape)
    fin.quant = "NONE"
    fin.data = x
    g.add(fin)
    g.add(graphs.Op("tpu.quant", "input_quant_i8", ["input"], x.shape, dict(scale=np.float32(128) / np.float32(t["input"]))))
    src = {o.name: o for o in g32.ops}

    def conv(name, inp, tx):
        o = src[name]
        wq, bq, rs, mu = Q.quantize_conv(o.weights["filter"], o.weights["bias"], tx, t[name])
        g.add(graphs.Op("tpu.conv_2d", name, [inp], o.shape, o.attrs, dict(filter=wq, bias=bq, rshift=rs, multiplier=mu),
                        "RSHIFT_AND_M_I32"))

    conv("c1", "input_quant_i8", t["input"])
    conv("c2", "c1", t["c1"])
    rs, mu = Q.quantize_rescale([t["c1"], t["c2"]], t["add"])
    g.add(graphs.Op("tpu.eltwise_add", "add", ["c1", "c2"], src["add"].shape, dict(do_relu=1),
                    dict(rshift=rs, multiplier=mu), "RSHIFT_AND_M_I8"))
    g.add(graphs.Op("tpu.pool_max_2d", "pool", ["add"], src["pool"].shape, src["pool"].attrs))
    g.add(graphs.Op("tpu.upsample", "up", ["pool"], src["up"].shape, src["up"].attrs))
    rs_c, mu_c = [], []
    for tx in (t["up"], t["c2"]):
        q = np.float32(tx) / np.float32(t["cat"])
        if abs(np.float32(t["cat"]) - np.float32(tx)) <= 1e-5:
            rs_c.append(0.0), mu_c.append(1.0)
        else:
            r, m = Q.find_rshift_and_multiplier(float(q))
            rs_c.append(float(r)), mu_c.append(float(m))
    g.add(graphs.Op("tpu.concat", "cat", ["up", "c2"], src["cat"].shape, dict(axis=1, do_relu=0),
                    dict(rshift=np.array(rs_c, np.float32), multiplier=np.array(mu_c, np.float32)), "RSHIFT_AND_M_I8"))
    conv("c3", "cat", t["cat"])
    g.add(graphs.Op("tpu.leaky_relu", "leaky", ["c3"], src["leaky"].shape, dict(negative_slope=0.1),
                    Q.quantize_leaky_relu(0.1, t["c3"], t["leaky"]), "RSHIFT_AND_M_I8"))
    g.add(graphs.Op("tpu.sigmoid", "sig", ["leaky"], src["sig"].shape, {},
                    dict(table=Q.quantize_lut_table("sigmoid", t["leaky"], 1.0)), "LUT_INT8"))
    qs = float(np.float32(float(np.float32(t["leaky"])) * float(np.float32(1.0)) / np.float32(t["mul"]) / 127.0))
    r, m = Q.find_rshift_and_multiplier(qs, qdm=True)
    g.add(graphs.Op("tpu.eltwise_mul", "mul", ["leaky", "sig"], src["mul"].shape, dict(do_relu=0),
                    dict(rshift=np.array([r], np.float32), multiplier=np.array([m], np.float32)), "RSHIFT_AND_M_I32"))
    rs, mu = Q.quantize_rescale([t["mul"]], t["gap"], divisor=hw * hw)
    ga = dict(src["gap"].attrs, count_include_pad=1)
    g.add(graphs.Op("tpu.pool_avg_2d", "gap", ["mul"], src["gap"].shape, ga, dict(rshift=rs, multiplier=mu),
                    "RSHIFT_AND_M_I8"))
    g.add(graphs.Op("tpu.reshape", "flat", ["gap"], (n, 24)))
    wq, bq, rs, mu = Q.quantize_fc(src["fc"].weights["filter"], src["fc"].weights["bias"], t["gap"], t["fc"])
    g.add(graphs.Op("tpu.fully_connected", "fc", ["flat"], (n, 10), dict(do_relu=0),
                    dict(filter=wq, bias=bq, rshift=rs, multiplier=mu), "RSHIFT_AND_M_I32"))
    dq = graphs.Op("tpu.quant", "fc_dequant", ["fc"], (n, 10), dict(scale=np.float32(t["fc"]) / np.float32(128)))
    dq.quant = "NONE"
    g.add(dq)
    g.outputs = ["fc_dequant"]
    return g


def run_pass(tmp_path):
    g32, acts, x = small_network()
    thr = measured_thresholds(acts)
    path, table = write_inputs(tmp_path, g32, thr)
    out = tmp_path / "net_int8.mlir"
    missing = Q.quantize_files(path, table, out)
    return g32, acts, x, thr, out, missing


def test_quantized_files_hold_what_the_helpers_compute(tmp_path):
    g32, acts, x, thr, out, missing = run_pass(tmp_path)
    assert missing == []
    want = expected_int8_graph(g32, thr, x)
    ops, weights, returns = describe(out)
    # modes, parameter kinds, the quant ops at the two edges
    assert returns == ["fc_dequant"]
    assert ops["input"]["quant"] == "NONE" and ops["input_quant_i8"]["type"] == "tpu.quant"
    assert ops["fc_dequant"]["quant"] == "NONE"
    for op in want.ops:
        if op.type in ("tpu.input", "tpu.quant", "tpu.reshape"):
            continue
        assert ops[op.name]["quant"] == "INT8", op.name
        if op.param_type.startswith("RSHIFT"):
            assert ops[op.name]["param"] == op.param_type, op.name
    t = thresholds_after_import(thr)
    assert f32_attr(out, "input_quant_i8", "scale") == np.float32(128) / np.float32(t["input"])
    assert f32_attr(out, "fc_dequant", "scale") == np.float32(t["fc"]) / np.float32(128)
    for name in ("add", "up", "c3", "sig", "pool"):
        assert f32_attr(out, name, "threshold") == np.float32(t[name]), name
    assert "count_include_pad=1" in ops["gap"]["line"]
    # every tensor of the new weight file
    with np.load(tmp_path / "net_int8_weights.npz") as z:
        have = {k: z[k] for k in z.files}
    assert sorted(have) == sorted(weights)
    roles = {"rshift": "rshift", "multiplier": "multiplier", "rshift_pos": "rshift_pos", "multiplier_pos": "multiplier_pos",
             "rshift_neg": "rshift_neg", "multiplier_neg": "multiplier_neg"}
    checked = 0
    for op in want.ops:
        for role, arr in op.weights.items():
            arr = np.asarray(arr, np.float32).ravel()
            if role in roles:
                got = have["%s_%s" % (op.name, role)].ravel()
            elif role == "table":
                full = have[op.name + "_y0_table"]
                assert full.shape == (1, 32, 16, 16)
                assert all(np.array_equal(full.reshape(32, 256)[i], full.reshape(32, 256)[0]) for i in range(32))
                got = full.reshape(32, 256)[0]
            else:     # filter / bias: the old tensor name + a suffix
                key = [k for k in have if k.startswith("%s_%s_" % (op.name, role)) and k.endswith("quant")]
                assert len(key) == 1, (op.name, role, sorted(have))
                got = have[key[0]].ravel()
            assert np.array_equal(got, arr), (op.name, role)
            checked += 1
    assert checked >= 25
    # the integers are integers, in range
    for k, v in have.items():
        assert np.array_equal(v, np.rint(v)), k


def test_threshold_rules_and_table_formats(tmp_path):
    g32, acts, x = small_network()
    thr = measured_thresholds(acts)
    path, table = write_inputs(tmp_path, g32, thr)
    # an op missing from the table is reported, not fatal at import; sigmoid needs no entry
    lines = [l for l in open(table).read().splitlines() if not l.startswith(("sig ", "up "))]
    open(table, "w").write("\r\n".join(lines) + "\r\nweight c1_filter " + " ".join(["0.5"] * 16) + "\nbitwidth c1_filter 8\n")
    missing = Q.quantize_files(path, table, tmp_path / "o.mlir")
    assert missing == ["up"]
    ops, _, _ = describe(tmp_path / "o.mlir")
    # `up` still ends with its producer's threshold through the forward rule
    th = lambda n: f32_attr(tmp_path / "o.mlir", n, "threshold")
    assert th("up") == th("pool") == th("add") == np.float32(thr["pool"])
    assert th("sig") == np.float32(1.0)
    # per-channel filter thresholds from the table replace the measured maxima
    with np.load(tmp_path / "o_weights.npz") as z:
        key = [k for k in z.files if k.startswith("c1_filter_")][0]
        wq_forced = z[key]
    src = {o.name: o for o in g32.ops}
    t = thresholds_after_import(thr)
    want, _, _, _ = Q.quantize_conv(src["c1"].weights["filter"], src["c1"].weights["bias"], t["input"], t["c1"],
                                    filter_threshold=np.full(16, 0.5, np.float32))
    assert np.array_equal(wq_forced.ravel(), np.asarray(want).ravel())
    # a malformed line is an error that quotes it
    open(table, "a").write("c1 zero point five\n")
    with pytest.raises(capi.TpuHipError, match="required format.*zero point five"):
        Q.quantize_files(path, table, tmp_path / "o2.mlir")


def test_pass_refuses_what_it_cannot_quantise(tmp_path):
    g = graphs.Graph("bad", 0)
    xin = graphs.Op("tpu.input", "input", [], (1, 8, 4, 4))
    xin.quant = "NONE"
    xin.data = np.zeros((1, 8, 4, 4), np.float32)
    g.add(xin)
    fp32_op(g, "tpu.softmax", "sm", ["input"], (1, 8, 4, 4), dict(axis=1))
    g.outputs = ["sm"]
    path = tmp_path / "bad.mlir"
    mlir_text.write_mlir(g, path)
    open(tmp_path / "t", "w").write("input 1.0\nsm 1.0\n")
    with pytest.raises(capi.TpuHipError, match="no INT8 quantisation for tpu.softmax"):
        Q.quantize_files(path, tmp_path / "t", tmp_path / "o.mlir")
    # a pass-through op whose two sides disagree (relu fed by a value with two uses keeps both thresholds)
    g = graphs.Graph("bad2", 0)
    g.add(xin)
    fp32_op(g, "tpu.permute", "perm", ["input"], (1, 4, 4, 8), dict(order0=0, order1=2, order2=3, order3=1))
    fp32_op(g, "tpu.eltwise_max", "mx", ["input", "input"], (1, 8, 4, 4), dict(do_relu=0))
    g.outputs = ["perm", "mx"]
    mlir_text.write_mlir(g, path)
    open(tmp_path / "t", "w").write("input 2.0\nperm 1.0\nmx 2.0\n")
    Q.quantize_files(path, tmp_path / "t", tmp_path / "o.mlir")          # forward rule makes perm 2.0: fine
    assert f32_attr(tmp_path / "o.mlir", "perm", "threshold") == np.float32(2.0)
    with pytest.raises(capi.TpuHipError, match="cannot open"):
        Q.quantize_files(tmp_path / "nope.mlir", tmp_path / "t", tmp_path / "o.mlir")


def test_mul_const_and_swap_channel_through_the_pass(tmp_path):
    g = graphs.Graph("mc", 0)
    xin = graphs.Op("tpu.input", "input", [], (1, 3, 4, 4))
    xin.quant = "NONE"
    xin.data = np.zeros((1, 3, 4, 4), np.float32)
    g.add(xin)
    fp32_op(g, "tpu.swap_channel", "bgr", ["input"], (1, 3, 4, 4), dict(channel_order0=2, channel_order1=1, channel_order2=0))
    fp32_op(g, "tpu.mul_const", "scaled", ["bgr"], (1, 3, 4, 4), dict(const_val=-2.5, do_relu=0))
    g.outputs = ["scaled"]
    path = tmp_path / "mc.mlir"
    mlir_text.write_mlir(g, path)
    open(tmp_path / "t", "w").write("input 2.0\nbgr 1.5\nscaled 3.0\n")
    assert Q.quantize_files(path, tmp_path / "t", tmp_path / "o.mlir") == []
    out = tmp_path / "o.mlir"
    # the rules run in the reference's order: mul_const takes |const| times its input's threshold
    # as the table gave it (1.5), and only afterwards does the pass-through swap_channel take its
    # own input's (2.0); only the sign of the constant is left
    assert f32_attr(out, "bgr", "threshold") == np.float32(2.0)
    assert f32_attr(out, "scaled", "threshold") == np.float32(3.75)
    assert f32_attr(out, "scaled", "const_val") == np.float32(-1.0)
    assert f32_attr(out, "scaled_dequant", "scale") == np.float32(3.75) / np.float32(128)
    ops, _, _ = describe(out)
    assert ops["bgr"]["quant"] == ops["scaled"]["quant"] == "INT8"
    assert "channel_order0=2" in ops["bgr"]["line"] and "channel_order2=0" in ops["bgr"]["line"]


def test_dilate_and_reflection_pad_through_the_pass(tmp_path):
    g = graphs.Graph("dr", 0)
    xin = graphs.Op("tpu.input", "input", [], (1, 3, 4, 6))
    xin.quant = "NONE"
    xin.data = np.zeros((1, 3, 4, 6), np.float32)
    g.add(xin)
    fp32_op(g, "tpu.dilate", "holes", ["input"], (1, 3, 7, 11), dict(ins0=1, ins1=1, fill_constant=0))
    fp32_op(g, "tpu.reflection_pad", "mirror", ["input"], (1, 3, 4, 11), dict(pads0=2, pads1=3))
    g.outputs = ["holes", "mirror"]
    path, out = tmp_path / "dr.mlir", tmp_path / "o.mlir"
    mlir_text.write_mlir(g, path)
    open(tmp_path / "t", "w").write("input 2.0\nholes 2.0\nmirror 2.0\n")
    assert Q.quantize_files(path, tmp_path / "t", out) == []
    ops, weights, _ = describe(out)
    assert ops["holes"]["quant"] == ops["mirror"]["quant"] == "INT8"
    wfile = [f for f in os.listdir(tmp_path) if f.endswith(".npz") and f.startswith("o")]
    assert len(wfile) == 1, os.listdir(tmp_path)
    w = np.load(tmp_path / wfile[0])
    # one anti-diagonal 0/1 matrix per side, the size of that side's pad
    for i, k in enumerate((2, 3)):
        assert np.array_equal(w["mirror_select_%d" % i], np.fliplr(np.eye(k, dtype=np.float32)))
    # a pass-through op whose sides disagree is refused (dilate is one; the mirror op is not checked)
    open(tmp_path / "t", "w").write("input 2.0\nholes 1.0\nmirror 1.0\n")
    with pytest.raises(capi.TpuHipError, match="thresholds differ"):
        Q.quantize_files(path, tmp_path / "t", out)


REF_GRAPHS = ["conv", "conv_1_oc", "deconv", "fc", "eltwise_add", "avg_pool", "max_pool", "relu", "concat",
              "broadcast_mul", "permute", "pixel_shuffle", "reorg", "reverse", "tile", "crop"]


def prepare_reference_graph(name, tmp_path, rng):
    """copies the reference's fp32 op graph, gives it random weights under the file name it asks
    for and a calibration table with one random threshold per op"""
    text = open(os.path.join(REF_TESTS, name + ".mlir")).read()
    path = tmp_path / (name + ".mlir")
    open(path, "w").write(text)
    ops, weights, wfile = [], {}, None
    for line in capi.mlir_describe(path).splitlines():
        w = line.split(" ")
        if w[0] == "weight_file":
            wfile = w[1]
        elif w[0] == "weight":
            shape = [int(v) for v in w[3][1:-1].split(",") if v]
            weights[w[1]] = rng.normal(0, 0.2, shape).astype(np.float32)
        elif w[0] == "op":
            ops.append((w[1], w[2], [int(v) for v in next(t for t in w[3:] if t.startswith("["))[1:-1].split(",") if v]))
    if weights:
        np.savez(tmp_path / wfile, **weights)
    table = tmp_path / (name + "_table")
    with open(table, "w") as f:
        for _, op_name, _ in ops:
            f.write("%s %.5f\n" % (op_name, rng.uniform(0.8, 4.0)))
    return path, table, ops, weights


@pytest.mark.skipif(not os.path.isdir(REF_TESTS), reason="the reference's op-test graphs are not present")
@pytest.mark.parametrize("name", REF_GRAPHS)
def test_reference_fp32_op_graphs_go_through_the_pass(name, tmp_path):
    rng = np.random.default_rng(len(name))
    path, table, ops, weights = prepare_reference_graph(name, tmp_path, rng)
    out = tmp_path / (name + "_int8.mlir")
    assert Q.quantize_files(path, table, out) == []
    got, wnames, returns = describe(out)
    for type_, op_name, _ in ops:
        if type_ in ("tpu.input", "tpu.reshape"):
            continue
        assert got[op_name]["quant"] == "INT8", op_name
    # fp32 in, fp32 out: one quant op per input in use, one dequant per returned value
    assert all(got[r]["type"] == "tpu.quant" and r.endswith("_dequant") for r in returns)
    assert any(n.endswith("_quant_i8") for n in got)
    if wnames:
        with np.load(tmp_path / (name + "_int8_weights.npz")) as z:
            assert sorted(z.files) == sorted(wnames)
    # written text reads back to the same description (printer and reader agree)
    again = tmp_path / "again.mlir"
    open(again, "w").write(open(out).read())
    assert capi.mlir_describe(again) == capi.mlir_describe(out)


@pytest.mark.gpu
def test_quantized_files_run_bit_exact_and_track_the_fp32_network(tmp_path):
    g32, acts, x, thr, out, _ = run_pass(tmp_path)
    want_graph = expected_int8_graph(g32, thr, x)
    want = oracle_graph.run(want_graph)
    t = thresholds_after_import(thr)
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.load(str(out))
    m.set_tensor("input", x)
    m.invoke()
    for op in want_graph.ops:
        if op.name in ("input", "fc_dequant"):
            continue
        got = m.get_tensor_i8(op.name)
        assert np.array_equal(got, want[op.name].reshape(op.shape)), op.name
        if op.name in acts:
            ref = acts[op.name].numpy().reshape(op.shape)
            deq = got.astype(np.float64) * t[op.name] / 127.0
            cos = (deq * ref).sum() / np.sqrt((deq * deq).sum() * (ref * ref).sum())
            assert cos > 0.99, (op.name, cos)
    y = m.get_tensor("fc_dequant")
    assert np.array_equal(y, want["fc_dequant"])
    ref = acts["fc"].numpy()
    assert np.abs(y - ref).max() < 0.08 * thr["fc"]
    m.close()


def lrn_network():
    """conv + ReLU -> LRN: -> (fp32 graph, input, torch activations, the three inner thresholds)"""
    import torch
    import torch.nn.functional as F
    torch.manual_seed(5)
    rng = np.random.default_rng(5)
    n, hw, size, alpha, beta, k = 2, 10, 5, 2e-2, 0.75, 1.0
    x = torch.tensor(rng.normal(0, 1, (n, 4, hw, hw)).astype(np.float32))
    w, b = torch.randn(24, 4, 3, 3) * 0.5, torch.randn(24) * 0.3
    a1 = F.relu(F.conv2d(x, w, b, padding=1))
    one = alpha / size * a1 * a1
    pad = F.pad(one, (0, 0, 0, 0, (size - 1) // 2, size - 1 - (size - 1) // 2))
    two = sum(pad[:, j:j + 24] for j in range(size))
    three = (two + k) ** -beta
    y = F.local_response_norm(a1, size, alpha, beta, k)
    assert torch.allclose(y, a1 * three, atol=1e-5)
    g = graphs.Graph("lrn32", 0)
    xin = graphs.Op("tpu.input", "input", [], tuple(x.shape))
    xin.quant = "NONE"
    xin.data = x.numpy()
    g.add(xin)
    fp32_op(g, "tpu.conv_2d", "c1", ["input"], tuple(a1.shape), conv_attrs(3, 1, True),
            dict(filter=w.numpy(), bias=b.numpy()))
    parts = [float(one.max()), float(two.max()), float(three.max())]
    fp32_op(g, "tpu.lrn", "norm", ["c1"], tuple(a1.shape),
            dict(local_size=size, alpha=alpha, beta=beta, k=k, sum_rshift=0, lrn_rshift=0, quant_data0=0, quant_data1=0,
                 threshold_parts0=parts[0], threshold_parts1=parts[1], threshold_parts2=parts[2]))
    g.outputs = ["norm"]
    return g, x.numpy(), dict(input=x, c1=a1, norm=y), parts


def test_lrn_tables_and_fractions_from_the_pass(tmp_path):
    g, x, acts, parts = lrn_network()
    path = tmp_path / "lrn.mlir"
    mlir_text.write_mlir(g, path)
    thr = measured_thresholds(acts)
    open(tmp_path / "t", "w").write("".join("%s %.7g\n" % kv for kv in thr.items()))
    out = tmp_path / "lrn_int8.mlir"
    assert Q.quantize_files(path, tmp_path / "t", out) == []
    ops, weights, _ = describe(out)
    line = ops["norm"]["line"]
    attr = lambda key: int(re.search(r"\b%s=(-?\d+)" % key, line).group(1))
    # x / y ~ quant / 2^shift, shift as large as keeps the quantised numerator within 8 bits + 1
    r0, q0, r1, q1 = attr("sum_rshift"), attr("quant_data0"), attr("lrn_rshift"), attr("quant_data1")
    f32 = np.float32
    assert 0 < q0 <= 256 and abs(q0 / 2.0 ** r0 - f32(parts[0]) / f32(parts[1])) <= 0.5 / 2.0 ** r0 + 1e-7
    want1 = f32(thr["c1"]) * f32(parts[2]) / (f32(thr["norm"]) * 256.0)
    assert 0 < q1 <= 256 and abs(q1 / 2.0 ** r1 - want1) <= 0.5 / 2.0 ** r1 + 1e-7
    assert r0 == 15 or 2.0 ** (r0 + 1) >= 256.0 * parts[1] / parts[0]
    with np.load(tmp_path / "lrn_int8_weights.npz") as z:
        sq, pw = z["norm_sq_gen_weight"], z["norm_power_gen_weight"]
    assert sq.shape == pw.shape == (1, 32, 16, 16)
    sq, pw = sq.reshape(32, 256), pw.reshape(32, 256)
    assert (sq == sq[0]).all() and (pw == pw[0]).all()
    idx = np.arange(256)
    # squares of thx/128 * idx scaled to 256 per sq threshold; (sum + k)^-beta scaled to 256 per its threshold
    sq_real = np.minimum((thr["c1"] / 128.0 * idx) ** 2 * 2e-2 / 5 * 256.0 / parts[0], 255)
    pw_real = np.minimum((idx / (256.0 / parts[1]) + 1.0) ** -0.75 * 256.0 / parts[2], 255)
    assert np.abs(sq[0] - sq_real).max() <= 0.5 + 1e-3 and np.abs(pw[0] - pw_real).max() <= 0.5 + 1e-3
    assert sq[0][0] == 0 and np.all(np.diff(sq[0]) >= 0) and np.all(np.diff(pw[0]) <= 0)


@pytest.mark.gpu
def test_lrn_graph_quantised_and_run_tracks_torch(tmp_path):
    g, x, acts, parts = lrn_network()
    path = tmp_path / "lrn.mlir"
    mlir_text.write_mlir(g, path)
    thr = measured_thresholds(acts)
    open(tmp_path / "t", "w").write("".join("%s %.7g\n" % kv for kv in thr.items()))
    out = tmp_path / "lrn_int8.mlir"
    assert Q.quantize_files(path, tmp_path / "t", out) == []
    m = module()
    m.load(str(out))
    m.set_tensor("input", x)
    m.invoke()
    got = m.get_tensor("norm_dequant").astype(np.float64).ravel()
    ref = acts["norm"].numpy().astype(np.float64).ravel()
    cos = (got * ref).sum() / np.sqrt((got * got).sum() * (ref * ref).sum())
    assert cos > 0.995, cos
    assert np.abs(got - ref).max() < 0.06 * thr["norm"]
    m.close()


def single_op_graph(kind, rng):
    """-> (fp32 graph, {input name: array}, torch result): the op graphs of the reference's backend
    tests (conv.mlir, deconv.mlir, fc.mlir, eltwise_add.mlir, avg_pool.mlir) rebuilt at small sizes"""
    import torch
    import torch.nn.functional as F
    g = graphs.Graph(kind, 0)

    def inp(name, shape):
        op = graphs.Op("tpu.input", name, [], shape)
        op.quant = "NONE"
        op.data = rng.normal(0, 1, shape).astype(np.float32)
        g.add(op)
        return torch.tensor(op.data)

    w = lambda *shape: (rng.normal(0, 0.2, shape)).astype(np.float32)
    if kind == "conv":
        x, f, b = inp("data", (4, 3, 32, 32)), w(32, 3, 3, 3), w(32)
        y = F.conv2d(x, torch.tensor(f), torch.tensor(b), stride=2, padding=1)
        fp32_op(g, "tpu.conv_2d", "conv", ["data"], tuple(y.shape), conv_attrs(3, 1, False, stride=2), dict(filter=f, bias=b))
    elif kind == "deconv":
        x, f, b = inp("data", (2, 16, 9, 7)), w(24, 16, 4, 4), w(24)
        y = F.conv_transpose2d(x, torch.tensor(f).transpose(0, 1).contiguous(), torch.tensor(b), stride=2, padding=1)
        fp32_op(g, "tpu.deconv_2d", "deconv", ["data"], tuple(y.shape), conv_attrs(4, 1, False, stride=2),
                dict(filter=f, bias=b))
    elif kind == "fc":
        x, f, b = inp("data", (4, 96)), w(40, 96), w(40)
        y = F.linear(x, torch.tensor(f), torch.tensor(b))
        fp32_op(g, "tpu.fully_connected", "fc", ["data"], (4, 40), dict(do_relu=0), dict(filter=f, bias=b))
    elif kind == "eltwise_add":
        x0, x1 = inp("data0", (2, 24, 10, 9)), inp("data1", (2, 24, 10, 9))
        y = F.relu(x0 + x1)
        fp32_op(g, "tpu.eltwise_add", "add", ["data0", "data1"], (2, 24, 10, 9), dict(do_relu=1))
    else:
        x = inp("data", (2, 20, 12, 12))
        y = F.avg_pool2d(x, 3, 3)
        fp32_op(g, "tpu.pool_avg_2d", "avg", ["data"], tuple(y.shape),
                dict(kernel_h=3, kernel_w=3, stride_h=3, stride_w=3, padding_t=0, padding_b=0, padding_l=0,
                     padding_r=0, do_relu=0, count_include_pad=0))
    g.outputs = [g.ops[-1].name]
    return g, {o.name: o.data for o in g.ops if o.type == "tpu.input"}, y


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["conv", "deconv", "fc", "eltwise_add", "avg_pool"])
def test_single_op_graphs_quantised_and_run_track_torch(kind, tmp_path):
    """the reference's flow for its backend op tests (compile.sh): fp32 result -> thresholds =
    max |activation| -> quantise -> INT8 interpreter, compared with the fp32 result"""
    rng = np.random.default_rng(len(kind) + 5)
    g, xs, y = single_op_graph(kind, rng)
    path = tmp_path / (kind + ".mlir")
    mlir_text.write_mlir(g, path)
    with open(tmp_path / "table", "w") as f:
        for n, v in xs.items():
            f.write("%s %.6f\n" % (n, np.abs(v).max()))
        f.write("%s %.6f\n" % (g.outputs[0], float(y.abs().max())))
    out = tmp_path / (kind + "_int8.mlir")
    assert Q.quantize_files(path, tmp_path / "table", out) == []
    m = module()
    m.load(str(out))
    for n, v in xs.items():
        m.set_tensor(n, v)
    m.invoke()
    (ret,) = list(m.get_output_details())
    assert ret == g.outputs[0] + "_dequant"
    got = m.get_tensor(ret).astype(np.float64).ravel()
    ref = y.numpy().astype(np.float64).ravel()
    cos = (got * ref).sum() / np.sqrt((got * got).sum() * (ref * ref).sum())
    assert cos > 0.995, cos
    assert np.abs(got - ref).max() < 0.05 * np.abs(ref).max()
    m.close()
