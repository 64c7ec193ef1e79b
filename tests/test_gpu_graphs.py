"""GPU parity on whole graphs through the module API (C++ op classes +
ModuleInterpreter behind the C ABI): every tensor of every layer must equal the
oracle's, for the five benchmark configurations at their full sizes."""
import os

import numpy as np
import pytest

import oracle_graph
from tpu_compiler_amd import capi, graphs, module

pytestmark = pytest.mark.gpu


def check_through_files(g, x, want, tmp_path):
    """the same graph as files: written as TPU-dialect text + weight .npz, loaded by name like
    pymlir's module.load, and run the way the tpuc-interpreter tool runs (.npz in, .npz out)"""
    from tpu_compiler_amd import mlir_text
    path = tmp_path / (g.name + ".mlir")
    wfile = mlir_text.write_mlir(g, path)
    m = module()
    m.load(str(path))
    assert m.get_weight_file_path() == os.path.basename(wfile)
    import contextlib
    import io
    err = io.StringIO()
    with contextlib.redirect_stderr(err):
        m.dump()
    assert err.getvalue() == open(path).read()
    assert [(i["name"], i["type"], i["quant"]) for i in m.op_info] == [(o.name, o.type, o.quant) for o in g.ops]
    assert list(m.get_output_details()) == list(g.outputs)
    m.set_tensor(g.input_op().name, np.asarray(x, np.float32))
    m.invoke()
    for op in g.ops:
        w = want[op.name].reshape(op.shape)
        got = m.get_tensor(op.name) if w.dtype == np.float32 or op.quant == "UINT8" else m.get_tensor_i8(op.name)
        assert np.array_equal(got, w.astype(got.dtype)), op.name
    m.close()
    np.savez(tmp_path / "in.npz", **{g.input_op().name: np.asarray(x, np.float32)})
    m = module()
    m.interpret_files(path, tmp_path / "in.npz", tmp_path / "out.npz", tmp_path / "all.npz")
    m.close()
    with np.load(tmp_path / "out.npz") as z:
        assert sorted(z.files) == sorted(g.outputs)
        for name in g.outputs:
            assert z[name].dtype == np.float32 and z[name].shape == tuple(g.by_name[name].shape)
            assert np.array_equal(z[name], want[name].reshape(z[name].shape).astype(np.float32)), name
    with np.load(tmp_path / "all.npz") as z:
        assert sorted(z.files) == sorted(o.name for o in g.ops)
        for op in g.ops:
            assert np.array_equal(z[op.name], want[op.name].reshape(op.shape).astype(np.float32)), op.name


@pytest.mark.parametrize("cfg,kw", [("cfg1", {}), ("cfg2", dict(batch=2)), ("cfg3", dict(batch=1, hw=96)),
                                    ("cfg4", dict(batch=2, hw=96)), ("cfg5", dict(batch=1, hw=96))])
def test_configurations_loaded_from_files_match_the_oracle(tmp_path, cfg, kw):
    g = graphs.CONFIGS[cfg](**kw)
    x = g.input_op().data
    check_through_files(g, x, oracle_graph.run(g), tmp_path)


def run_and_compare(g, check_stats=True):
    m = module()
    try:
        m.load(g)
        inp = g.input_op()
        m.set_tensor(inp.name, inp.data.astype(np.float32))
        m.invoke()
        guards = {}
        want = oracle_graph.run(g, guards=guards if g.input_op().shape[0] <= 8 else None)
        bad = []
        for op in g.ops:
            got = m.get_tensor_i8(op.name)
            ref = want[op.name].reshape(got.shape)
            if not np.array_equal(got, ref):
                bad.append((op.name, op.type, int((got != ref).sum()), got.size))
        assert not bad, "mismatching layers (name, type, wrong, total): %s" % bad[:8]
        for name, gv in guards.items():
            assert gv < (1 << 24), "fp32-exactness guard broken at %s: %d" % (name, gv)
        if check_stats:
            # the comparison must not be trivially true: activations are alive everywhere
            for op in g.ops:
                if op.type in ("tpu.conv_2d", "tpu.fully_connected", "tpu.eltwise_add"):
                    y = want[op.name]
                    assert len(np.unique(y)) > 16, op.name
                    assert np.mean(y == 0) < 0.9, op.name
        return m, want
    except Exception:
        m.close()
        raise


def test_cfg1_single_conv():
    g = graphs.cfg1_single_conv()
    m, want = run_and_compare(g)
    # float view of the same tensor, as the reference hands it out
    f = m.get_tensor("conv")
    assert f.dtype == np.float32 and np.array_equal(f, want["conv"].astype(np.float32))
    assert dict(m.kernels())["conv"].startswith("mfma")
    m.close()


def test_cfg2_mobilenet_block():
    g = graphs.cfg2_mobilenet_block()
    m, _ = run_and_compare(g)
    k = dict(m.kernels())
    assert k["dw"] == "depthwise" and k["pw"].startswith("mfma")
    m.close()


def test_cfg3_resnet50_batch32():
    g = graphs.cfg3_resnet50()
    assert len(g.conv_ops()) == 54 and g.input_op().shape == (32, 3, 224, 224)
    m, want = run_and_compare(g)
    assert want["fc1000"].shape == (32, 1000)
    m.close()


def test_cfg4_mobilenet_v2_batch64():
    g = graphs.cfg4_mobilenet_v2()
    assert g.input_op().shape == (64, 3, 224, 224)
    m, _ = run_and_compare(g)
    m.close()


def test_cfg5_yolo_v3_batch8():
    g = graphs.cfg5_yolo_v3()
    assert g.input_op().shape == (8, 3, 608, 608) and len(g.outputs) == 3
    m, want = run_and_compare(g)
    assert [want[o].shape for o in g.outputs] == [(8, 255, 19, 19), (8, 255, 38, 38),
                                                  (8, 255, 76, 76)]
    m.close()


def test_module_api_semantics():
    """batch slots, invoke_to, run(), get_all_tensor, reload keeps clean kernels."""
    g = graphs.cfg3_resnet50(batch=1, hw=64)
    m = module(max_batch=2)
    m.load(g)
    assert list(m.get_input_details()) == ["input"]
    assert m.get_input_details()["input"] == 3 * 64 * 64
    assert m.get_output_details() == ["fc1000"]
    assert m.tensor_dtype("conv1") == "INT8"
    assert m.tensor_shape("pool5_flat") == (1, 2048)
    import contextlib
    import io
    err = io.StringIO()
    with contextlib.redirect_stderr(err):
        m.dump()
    assert "tpu.conv_2d conv1 INT8" in err.getvalue() and err.getvalue().count("\n") == len(g.ops)
    with pytest.raises(NotImplementedError):
        m.set_plugin("plugin.so")
    x0 = g.input_op().data
    x1 = np.ascontiguousarray(x0[:, :, ::-1, :])
    want0 = oracle_graph.run(g)
    want1 = oracle_graph.run(g, input_data=x1)
    # slot 1 and slot 0 are independent runs of the N=1 graph
    m.set_tensor("input", x1.astype(np.float32), 1)
    m.set_tensor("input", x0.astype(np.float32), 0)
    m.invoke(1)
    m.invoke(0)
    assert np.array_equal(m.get_tensor_i8("fc1000", 1), want1["fc1000"])
    assert np.array_equal(m.get_tensor_i8("fc1000", 0), want0["fc1000"])
    # fastInvokeAllBatch runs every dirty kernel for each slot
    m2 = module(max_batch=2)
    m2.load(g)
    m2.set_tensor("input", x0.astype(np.float32), 0)
    m2.set_tensor("input", x1.astype(np.float32), 1)
    m2.fast_invoke_all_batch("", 2)
    assert np.array_equal(m2.get_tensor_i8("res3a", 1), want1["res3a"])
    assert np.array_equal(m2.get_tensor_i8("res3a", 0), want0["res3a"])
    m2.close()
    # run(): flat float array in, dict of outputs out; target_op stops early
    out = m.run(x0.astype(np.float32))
    assert list(out) == ["fc1000"] and np.array_equal(out["fc1000"], want0["fc1000"])
    out = m.run(x0.astype(np.float32), "res2a")
    assert np.array_equal(out["res2a"], want0["res2a"].astype(np.float32))
    allt = m.get_all_tensor()
    assert set(allt) == {op.name for op in g.ops}
    # reload with one op changed: only it and its consumers are rebuilt (dirty check)
    g.by_name["res5c_branch2c"].attrs["do_relu"] = 1
    m.load(g)
    m.invoke(0)
    want2 = oracle_graph.run(g)
    assert np.array_equal(m.get_tensor_i8("fc1000", 0), want2["fc1000"])
    assert not np.array_equal(want2["res5c_branch2c"], want0["res5c_branch2c"])
    m.close()


def test_partial_reload_of_fused_and_paired_kernels_after_fast_invoke():
    """fastInvokeAllBatch clears the dirty flags; a reload that rebuilds only the add fused into a
    retained conv, the second conv of a pair, or its first, must run the launch that writes the
    rebuilt kernel's fresh result tensor (MlirModuleInterpreter.cpp:85-116, 383-405)."""
    g = graphs.cfg3_resnet50(batch=1, hw=64)
    x = g.input_op().data.astype(np.float32)
    m = module(max_batch=1)
    m.load(g)
    m.set_tensor("input", x, 0)
    m.fast_invoke_all_batch("", 1)
    kern = dict(m.kernels())
    assert kern["res3a_branch2a"] == "with res3a_branch1", kern["res3a_branch2a"]
    want = oracle_graph.run(g)
    assert np.array_equal(m.get_tensor_i8("fc1000", 0), want["fc1000"])
    for name, attr in (("res2b", "do_relu"),               # the add folded into res2b_branch2c
                       ("res3a_branch2a", "do_relu"),      # second conv of a pair
                       ("res4a_branch1", "do_relu"),       # first conv of a pair
                       ("res5c", "do_relu")):
        g.by_name[name].attrs[attr] = 0 if g.by_name[name].attrs.get(attr, 0) else 1
        m.load(g)
        m.fast_invoke_all_batch("", 1)
        want = oracle_graph.run(g)
        for op in g.ops:
            assert np.array_equal(m.get_tensor_i8(op.name, 0), want[op.name].reshape(op.shape)), (name, op.name)
    m.close()


def test_fusion_on_and_off_give_the_same_tensors(monkeypatch):
    g = graphs.cfg3_resnet50(batch=2, hw=96)
    want = oracle_graph.run(g)
    for fuse in ("1", "0"):
        monkeypatch.setenv("TPUHIP_FUSE", fuse)
        m = module()
        m.load(g)
        m.set_tensor("input", g.input_op().data.astype(np.float32))
        m.invoke()
        for op in g.ops:
            assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), \
                (fuse, op.name)
        m.close()


def test_sibling_convs_run_as_one_launch_with_unchanged_results():
    """the projection shortcut and the first 1x1 conv of a downsampling block read the same tensor
    through the same window: one launch serves both.  On, off, reloaded and stopped half way, every
    tensor equals the oracle's."""
    g = graphs.cfg3_resnet50(batch=2, hw=96)
    want = oracle_graph.run(g)
    pairs = [("res%da_branch1" % s, "res%da_branch2a" % s) for s in (2, 3, 4, 5)]
    for on in (1, 0):
        m = module()
        m.set_option("pair_convs", on)
        m.load(g)
        algo = dict(m.kernels())
        for first, second in pairs:
            assert algo[first].startswith("mfma")
            assert algo[second] == ("with " + first if on else algo[second]) and (on or algo[second].startswith("mfma"))
        times = {name: ms for name, _, ms in m.time_kernels(iters=2)}
        if on:
            assert all(times[second] == 0 and times[first] > 0 for first, second in pairs)
        m.set_tensor("input", g.input_op().data.astype(np.float32))
        m.invoke()
        for op in g.ops:
            assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), (on, op.name)
        if on:
            # a reload keeps the pairing; stopping at the second conv of a pair still produces it
            m.load(g)
            assert dict(m.kernels())["res3a_branch2a"] == "with res3a_branch1"
            m.set_tensor("input", g.input_op().data.astype(np.float32))
            m.invoke_to("res3a_branch2a")
            assert np.array_equal(m.get_tensor_i8("res3a_branch2a"),
                                  want["res3a_branch2a"].reshape(g.by_name["res3a_branch2a"].shape))
        m.close()


def test_a_stem_that_took_its_max_pool_is_left_out_of_pairing():
    """two 7x7 / stride 2 convs over the image, the first with 128 output channels (a candidate first of a
    pair), the second a stem with its max pool folded into its launch: pairing must not swallow the stem, or
    the pooled tensor would never be written.  Also: with two readers, one of them off the stem path, the
    image keeps its 16-byte channel stride."""
    from tpu_compiler_amd.graphs import Builder, BASE_SEED
    b = Builder("sibling_stems", BASE_SEED + 77, 2, (6, 16))
    x = b.input("input", 3, 64, 64)
    wide = b.conv("wide", x, 128, 7, stride=2, pad=3, relu=True)
    stem = b.conv("stem", x, 64, 7, stride=2, pad=3, relu=True)
    pooled = b.pool_max("pool", stem, 3, 2, (0, 1, 0, 1))
    g = b.finish([wide, pooled])
    want = oracle_graph.run(g)
    for keep in (1, 0):
        m = module()
        m.set_option("keep_all_tensors", keep)
        m.load(g)
        algo = dict(m.kernels())
        assert algo["stem"] == "stem" and not algo["wide"].startswith("with")
        m.set_tensor("input", g.input_op().data.astype(np.float32))
        m.invoke()
        for name in ("wide", "pool") + (("stem",) if keep else ()):
            assert np.array_equal(m.get_tensor_i8(name), want[name].reshape(g.by_name[name].shape)), (keep, name)
        m.close()


def test_chained_pointwise_convs_run_as_one_launch_with_unchanged_results():
    """the 1x1 expansion + add that closes a bottleneck block and the 1x1 reduction that opens the next
    run as one launch (res2a/b, res3a/b/c of the ResNet-50 shape).  On, off, with every tensor kept and
    with outputs only, reloaded, partially reloaded and stopped at the second conv of a chain, every
    tensor written equals the oracle's."""
    g = graphs.cfg3_resnet50(batch=2, hw=96)
    want = oracle_graph.run(g)
    chains = [("res2a_branch2c", "res2b_branch2a"), ("res2b_branch2c", "res2c_branch2a"),
              ("res3a_branch2c", "res3b_branch2a"), ("res3b_branch2c", "res3c_branch2a"),
              ("res3c_branch2c", "res3d_branch2a")]
    x = g.input_op().data.astype(np.float32)
    for on, keep in ((1, 1), (1, 0), (0, 1)):
        m = module()
        m.set_option("chain_convs", on)
        m.set_option("keep_all_tensors", keep)
        m.load(g)
        algo = dict(m.kernels())
        for first, second in chains:
            assert algo[first].startswith("mfma_chain_") == bool(on), (on, first, algo[first])
            assert (algo[second] == "with " + first) == bool(on), (on, second, algo[second])
        times = {name: ms for name, _, ms in m.time_kernels(iters=2)}
        if on:
            assert all(times[second] == 0 and times[first] > 0 for first, second in chains)
        m.set_tensor("input", x)
        m.invoke()
        for op in g.ops:
            try:
                got = m.get_tensor_i8(op.name)
            except capi.TpuHipError as e:
                assert not keep and "never written" in str(e)
                continue
            assert np.array_equal(got, want[op.name].reshape(op.shape)), (on, keep, op.name)
        if on and keep:
            # a reload keeps the chains; stopping at the second conv of a chain still produces it
            m.load(g)
            assert dict(m.kernels())["res3b_branch2a"] == "with res3a_branch2c"
            m.set_tensor("input", x)
            m.invoke_to("res3b_branch2a")
            assert np.array_equal(m.get_tensor_i8("res3b_branch2a"),
                                  want["res3b_branch2a"].reshape(g.by_name["res3b_branch2a"].shape))
        m.close()
    # partial reloads after fast_invoke_all_batch: only the second conv, the add in the middle, or the
    # first conv of a chain is rebuilt; the launch that writes the rebuilt kernel's tensor must run
    g = graphs.cfg3_resnet50(batch=1, hw=64)
    m = module(max_batch=1)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32), 0)
    m.fast_invoke_all_batch("", 1)
    for name in ("res2b_branch2a", "res2a", "res3b_branch2c"):
        g.by_name[name].attrs["do_relu"] = 0 if g.by_name[name].attrs.get("do_relu", 0) else 1
        m.load(g)
        m.fast_invoke_all_batch("", 1)
        want = oracle_graph.run(g)
        for op in g.ops:
            assert np.array_equal(m.get_tensor_i8(op.name, 0), want[op.name].reshape(op.shape)), (name, op.name)
    m.close()


@pytest.mark.parametrize("builder,kw,first", [(graphs.cfg3_resnet50, dict(batch=2, hw=96), "conv1"),
                                              (graphs.cfg4_mobilenet_v2, dict(batch=2, hw=64), "conv1"),
                                              (graphs.cfg5_yolo_v3, dict(batch=1, hw=96), "conv1")])
def test_three_channel_graph_input_packed_to_one_dword_per_pixel(builder, kw, first):
    """the image input of the networks, read only by the stem conv, lies at a channel stride of 4 by default
    and 16 with the option off: every tensor equals the oracle's either way, the input reads back as it
    was set, and a reload that changes nothing keeps the layout"""
    g = builder(**kw)
    want = oracle_graph.run(g)
    x = g.input_op().data.astype(np.float32)
    for on in (1, 0):
        m = module()
        m.set_option("pack_inputs", on)
        m.load(g)
        assert dict(m.kernels())[first] == "stem"
        for _ in range(2):
            m.set_tensor("input", x)
            m.invoke()
            assert np.array_equal(m.get_tensor_i8("input"), g.input_op().data.reshape(g.input_op().shape))
            for op in g.ops:
                assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), (on, op.name)
            m.load(g)
        m.close()


@pytest.mark.parametrize("builder,kw", [(graphs.cfg5_yolo_v3, dict(batch=1, hw=96)),
                                        (graphs.cfg4_mobilenet_v2, dict(batch=2, hw=64)),
                                        (graphs.cfg2_mobilenet_block, dict(batch=1))])
def test_table_fusion_on_off_and_outputs_only_agree_with_the_oracle(monkeypatch, builder, kw):
    """leaky-relu / clip tables ride in the producing conv; every variant gives the oracle's bytes"""
    g = builder(**kw)
    want = oracle_graph.run(g)
    for fuse, keep in (("1", 1), ("0", 1), ("1", 0)):
        monkeypatch.setenv("TPUHIP_FUSE", fuse)
        m = module()
        m.set_option("keep_all_tensors", keep)
        m.load(g)
        m.set_tensor("input", g.input_op().data.astype(np.float32))
        m.invoke()
        launched = [a for _, a in m.kernels()]
        checked = 0
        for op in g.ops:
            try:
                got = m.get_tensor_i8(op.name)
            except capi.TpuHipError as e:
                assert keep == 0 and "never written" in str(e), (op.name, str(e))
                continue
            assert np.array_equal(got, want[op.name].reshape(op.shape)), (fuse, keep, op.name)
            checked += 1
        for name in g.outputs:
            assert np.array_equal(m.get_tensor_i8(name), want[name].reshape(g.by_name[name].shape))
        assert checked == len(g.ops) if keep else checked < len(g.ops)
        m.close()


def test_outputs_only_mode_skips_fused_conv_results_and_keeps_the_rest_exact():
    g = graphs.cfg3_resnet50(batch=2, hw=96)
    want = oracle_graph.run(g)
    m = module()
    m.set_option("keep_all_tensors", 0)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    adds = [op for op in g.ops if op.type == "tpu.eltwise_add"]
    consumers = {}
    for op in g.ops:
        for i in op.inputs:
            consumers.setdefault(i, []).append(op.name)
    skipped = 0
    for op in g.ops:
        only = g.by_name[consumers[op.name][0]] if len(consumers.get(op.name, [])) == 1 else None
        fused_away = op.type == "tpu.conv_2d" and only is not None and (
            (only.type == "tpu.eltwise_add" and only.inputs[-1] == op.name)
            or (only.type == "tpu.pool_max_2d" and op.name == "conv1"))   # the stem's pool rides in its launch
        if fused_away:
            with pytest.raises(capi.TpuHipError, match="never written"):
                m.get_tensor_i8(op.name)
            skipped += 1
        else:
            assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    assert len(adds) == 16 and skipped == 17
    assert dict(m.kernels())["conv1"] == "stem"
    with pytest.raises(capi.TpuHipError, match="unknown option"):
        m.set_option("nope", 1)
    # back to the default: everything readable again after a reload
    m.set_option("keep_all_tensors", 1)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    m.close()


def test_benchmark_configuration_full_size_against_the_oracle():
    """exactly what bench.py times by default: cfg3 at batch 32, the recorded conv tile variants,
    outputs-only mode -- every tensor that is written, and fc1000, must equal the oracle's"""
    import json
    import os
    import bench
    g = graphs.cfg3_resnet50()
    tiles = json.load(open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                        bench.RECORDED_TILES["cfg3"])))
    lib = capi.bind()
    names = []
    while lib.tpuhip_conv2d_tile_name(len(names)):
        names.append(lib.tpuhip_conv2d_tile_name(len(names)).decode())
    for name, algo in tiles.items():
        if algo in names:      # (a layer that opens a chained launch is recorded under that kernel's name)
            g.by_name[name].attrs["algo"] = 16 + names.index(algo)
    want = oracle_graph.run(g)
    m = module()
    m.set_option("keep_all_tensors", 0)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    kern = dict(m.kernels())
    for name, algo in tiles.items():
        assert kern[name] == algo or kern[name].startswith("with "), (name, kern[name], algo)
    assert sum(1 for a in kern.values() if a.startswith("mfma_chain_")) == 5   # res2a/b, res3a/b/c open a chain
    written = skipped = 0
    for op in g.ops:
        try:
            got = m.get_tensor_i8(op.name)
        except capi.TpuHipError as e:
            assert "never written" in str(e)
            skipped += 1
            continue
        assert np.array_equal(got, want[op.name].reshape(op.shape)), op.name
        written += 1
    # 16 conv results go straight into their fused add, conv1 into its fused max pool
    assert skipped == 17 and written == len(g.ops) - 17
    assert np.array_equal(m.get_tensor_i8("fc1000"), want["fc1000"])
    m.close()


def test_int8_host_entry_sets_the_same_tensor_as_the_float_one():
    g = graphs.cfg3_resnet50(batch=2, hw=64)
    x = g.input_op().data
    m = module()
    m.load(g)
    m.set_tensor("input", x.astype(np.float32))
    m.invoke()
    want = {k: m.get_tensor_i8(k) for k in ("input", "fc1000")}
    m.set_tensor("input", np.zeros(x.shape, np.float32))
    m.set_tensor_i8("input", x)
    m.invoke()
    for k, v in want.items():
        assert np.array_equal(m.get_tensor_i8(k), v), k
    with pytest.raises(capi.TpuHipError, match="size mismatch"):
        m.set_tensor_i8("input", x[:1])
    with pytest.raises(TypeError):
        m.set_tensor_i8("input", x.astype(np.float32))
    m.close()


@pytest.mark.parametrize("shape,order", [
    ((2, 3, 4, 5, 7), (0, 2, 1, 3, 4)),        # the channel-shuffle form [N, g, C/g, H, W]
    ((1, 2, 2, 3, 4, 5), (0, 3, 4, 1, 5, 2)),  # the pixel-shuffle form, 6-d: not foldable to 4-d
    ((3, 2, 5, 4, 6), (4, 0, 3, 1, 2)),
    ((4, 5, 6), (2, 0, 1)),
    ((7, 9), (1, 0)),
])
def test_permute_of_shapes_that_are_not_4d(shape, order):
    """PermuteOpKernel on ranks 2, 3, 5, 6 (the reference folds them to 4-d where it can,
    parsePermuteParam) between reshapes, against numpy's transpose"""
    rng = np.random.default_rng(sum(shape))
    size = int(np.prod(shape))
    flat4 = (shape[0], size // shape[0], 1, 1)
    x = rng.integers(-128, 128, flat4).astype(np.int8)
    out_shape = tuple(shape[o] for o in order)
    g = graphs.Graph("permute_nd", 3)
    g.add(graphs.Op("tpu.input", "input", [], flat4)).data = x
    g.add(graphs.Op("tpu.reshape", "nd", ["input"], shape))
    g.add(graphs.Op("tpu.permute", "perm", ["nd"], out_shape, {"order%d" % d: o for d, o in enumerate(order)}))
    g.add(graphs.Op("tpu.reshape", "back", ["perm"], (out_shape[0], size // out_shape[0], 1, 1)))
    g.outputs = ["back"]
    want = np.transpose(x.reshape(shape), order)
    assert np.array_equal(oracle_graph.run(g)["perm"], want)
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.load(g)
    m.set_tensor("input", x.astype(np.float32))
    m.invoke()
    assert np.array_equal(m.get_tensor_i8("perm").reshape(out_shape), want)
    assert np.array_equal(m.get_tensor_i8("back").reshape(-1), want.reshape(-1))
    m.close()


def test_channel_shuffle_written_as_reshape_permute_reshape_equals_the_shuffle_op():
    rng = np.random.default_rng(8)
    n, c, h, w, grp = 2, 24, 6, 5, 3
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    g = graphs.Graph("shuffle_nd", 4)
    g.add(graphs.Op("tpu.input", "input", [], x.shape)).data = x
    g.add(graphs.Op("tpu.reshape", "r5", ["input"], (n, grp, c // grp, h, w)))
    g.add(graphs.Op("tpu.permute", "p5", ["r5"], (n, c // grp, grp, h, w),
                    {"order0": 0, "order1": 2, "order2": 1, "order3": 3, "order4": 4}))
    g.add(graphs.Op("tpu.reshape", "r4", ["p5"], x.shape))
    g.add(graphs.Op("tpu.shuffle_channel", "sc", ["input"], x.shape, dict(group=grp)))
    g.outputs = ["r4", "sc"]
    m = module()
    m.load(g)
    m.set_tensor("input", x.astype(np.float32))
    m.invoke()
    a, b = m.get_tensor_i8("r4"), m.get_tensor_i8("sc")
    assert np.array_equal(a, b) and np.array_equal(a, oracle_graph.run(g)["sc"])
    m.close()


def test_module_errors_are_reported():
    g = graphs.cfg1_single_conv()
    m = module()
    m.load(g)
    with pytest.raises(capi.TpuHipError, match="size"):
        m.set_tensor("input", np.zeros(10, np.float32))
    with pytest.raises(capi.TpuHipError, match="Not Find"):
        m.get_tensor_i8("nope")
    bad = np.zeros(g.input_op().shape, np.float32)
    bad[0, 0, 0, 0] = 0.5
    with pytest.raises(capi.TpuHipError, match="int8"):
        m.set_tensor("input", bad)
    g2 = graphs.cfg1_single_conv()
    g2.ops[1].type = "tpu.softmax"
    with pytest.raises(capi.TpuHipError, match="no support"):
        module().load(g2)
    g3 = graphs.cfg1_single_conv()
    del g3.ops[1].weights["multiplier"]
    with pytest.raises(capi.TpuHipError, match="multiplier"):
        module().load(g3)
    g4 = graphs.cfg1_single_conv()
    g4.ops[1].quant = "BF16"
    with pytest.raises(capi.TpuHipError, match="INT8"):
        module().load(g4)
    m.close()


def test_lut_activation_and_general_reshape():
    """a y0-table activation (sigmoid-style op) and a reshape that is not an alias in
    channels-last order."""
    b = graphs.Builder("lut_reshape", 77, 2, (4, 18))
    x = b.input("input", 24, 5, 6)
    y = b.conv("conv", x, 40, 3, relu=False)
    g = b.finish([y])
    table = np.clip(np.rint(127 / (1 + np.exp(-np.arange(-128, 128) / 16.0))), -128, 127)
    table = np.roll(table, 128).astype(np.float32)   # entry i <-> two's-complement byte i
    g.add(graphs.Op("tpu.sigmoid", "sig", ["conv"], g.by_name["conv"].shape, {},
                    {"table": table}, "LUT_INT8"))
    g.add(graphs.Op("tpu.reshape", "flat", ["sig"], (2, 40 * 5 * 6)))
    g.add(graphs.Op("tpu.reshape", "back", ["flat"], (2, 8, 25, 6)))
    g.outputs = ["back"]
    m = module()
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    conv = oracle_graph.run(g, upto="conv")["conv"]
    import oracle_lib as O
    sig = O.lut_i8(conv, table)
    assert np.array_equal(m.get_tensor_i8("sig"), sig)
    assert np.array_equal(m.get_tensor_i8("flat"), sig.reshape(2, -1))
    assert np.array_equal(m.get_tensor_i8("back"), sig.reshape(2, 8, 25, 6))
    m.close()


def test_graph_with_elementwise_family_matches_the_oracle(tmp_path):
    """a squeeze-excite shaped graph: conv pair -> max / min / mul -> global average ->
    1x1 conv gate -> broadcast mul / add / sub with the feature map"""
    b = graphs.Builder("se_block", graphs.BASE_SEED + 77, 2, (6, 12))
    x = b.input("input", 24, 12, 10)
    c1 = b.conv("c1", x, 40, 3, relu=True)
    c2 = b.conv("c2", x, 40, 3, relu=False)
    g = b.g
    shp = g.by_name[c1].shape
    f32 = lambda *v: np.array(v, np.float32)

    def binop(t, name, srcs, shape, mult, rshift, relu=0):
        g.add(graphs.Op(t, name, srcs, shape, dict(do_relu=relu),
                        dict(rshift=f32(rshift), multiplier=f32(*mult)), "RSHIFT_AND_M_I8"))
        return name

    slope = (np.arange(shp[1]) % 23 - 7).astype(np.float32)
    g.add(graphs.Op("tpu.prelu", "pr", [c2], shp, {},
                    dict(slope=slope, rshift_pos=f32(1), multiplier_pos=f32(3), rshift_neg=f32(3)),
                    "RSHIFT_AND_M_I8"))
    mx = binop("tpu.eltwise_max", "mx", [c1, c2], shp, (3, 2), 1)
    mn = binop("tpu.eltwise_min", "mn", [c1, "pr"], shp, (1, 1), 0, relu=1)
    ml = binop("tpu.eltwise_mul", "ml", [mx, mn], shp, (1518500250,), 6)
    g.add(graphs.Op("tpu.pool_avg_2d", "gap", ["ml"], (shp[0], shp[1], 1, 1),
                    dict(kernel_h=shp[2], kernel_w=shp[3], stride_h=1, stride_w=1, padding_t=0,
                         padding_b=0, padding_l=0, padding_r=0, do_relu=0),
                    dict(rshift=f32(7), multiplier=f32(2)), "RSHIFT_AND_M_I8"))
    pooled = "gap"
    gate = binop("tpu.broadcast_mul", "gate", [mx, pooled], shp, (1 << 30,), 5)
    ba = binop("tpu.broadcast_add", "badd", [gate, pooled], shp, (2, 3), 2, relu=1)
    bs = binop("tpu.broadcast_sub", "bsub", [pooled, ba], shp, (9, 5), 1)
    g.outputs = [bs]
    want = oracle_graph.run(g)
    m = module()
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    assert len(np.unique(want[bs])) > 8
    m.close()
    check_through_files(g, g.input_op().data, want, tmp_path)


def test_graph_with_data_movement_ops_matches_the_oracle(tmp_path):
    b = graphs.Builder("movers", graphs.BASE_SEED + 78, 2, (6, 12))
    x = b.input("input", 12, 8, 6)
    c1 = b.conv("c1", x, 36, 3, relu=True)
    g = b.g

    def mv(t, name, src, shape, **attrs):
        g.add(graphs.Op(t, name, [src], shape, attrs))
        return name

    n = 2
    p = mv("tpu.pad", "pad", c1, (n, 36, 11, 9), pads0=0, pads1=0, pads2=1, pads3=2, pads4=0, pads5=0,
           pads6=2, pads7=1)
    pe = mv("tpu.pad", "pad_edge", c1, (n, 36, 10, 8), mode_edge=1, pads0=0, pads1=0, pads2=1, pads3=1,
            pads4=0, pads5=0, pads6=1, pads7=1)
    cr = mv("tpu.crop", "crop", p, (n, 20, 8, 6), crop_offset0=0, crop_offset1=4, crop_offset2=1,
            crop_offset3=2)
    pm = mv("tpu.permute", "perm", cr, (n, 8, 6, 20), order0=0, order1=2, order2=3, order3=1)
    ro = mv("tpu.reorg", "reorg", c1, (n, 144, 4, 3), stride=2)
    d2s = mv("tpu.pixelshuffle", "d2s", ro, (n, 36, 8, 6), upscale_factor=2, mode_dcr=1)
    tl = mv("tpu.tile", "tile", d2s, (n, 36, 8, 18), axis=3, tiles=3)
    rv = mv("tpu.reverse", "rev", tl, (n, 36, 8, 18), axis=2)
    sh = mv("tpu.shuffle_channel", "shuf", rv, (n, 36, 8, 18), group=4)
    g.outputs = [pm, pe, sh]
    want = oracle_graph.run(g)
    # DCR depth-to-space undoes a reorg (both put the block offset outermost in the channels)
    assert np.array_equal(want["d2s"], want["c1"])
    m = module()
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    m.close()
    check_through_files(g, g.input_op().data, want, tmp_path)


@pytest.mark.parametrize("fuse", [1, 0])
def test_graph_with_swap_channel_mul_const_and_zero_mask(tmp_path, fuse):
    """BGR<->RGB swap in front of a stem conv, then the two byte-wise ops that run as tables
    (fused into the conv in front of them when fusion is on)"""
    b = graphs.Builder("byte_ops", graphs.BASE_SEED + 81, 2, (6, 12))
    x = b.input("input", 3, 18, 14)
    g = b.g
    g.add(graphs.Op("tpu.swap_channel", "bgr", [x], g.by_name[x].shape,
                    dict(channel_order0=2, channel_order1=1, channel_order2=0)))
    b.cal["bgr"] = b.cal[x][:, [2, 1, 0]]
    c1 = b.conv("c1", "bgr", 24, 3, relu=False)
    c2 = b.conv("c2", "bgr", 24, 3, relu=False)
    shp = g.by_name[c1].shape
    g.add(graphs.Op("tpu.mul_const", "neg", [c1], shp, dict(const_val=-1.0, do_relu=1)))
    g.add(graphs.Op("tpu.zero_mask", "mask", [c2], shp, dict(positive=1)))
    g.add(graphs.Op("tpu.zero_mask", "hole", ["neg"], shp, dict(positive=0)))
    g.add(graphs.Op("tpu.eltwise_min", "both", ["mask", "hole"], shp, dict(do_relu=0),
                    dict(rshift=np.array([0], np.float32), multiplier=np.array([1, 1], np.float32)),
                    "RSHIFT_AND_M_I8"))
    g.outputs = ["both", "neg"]
    want = oracle_graph.run(g)
    assert np.array_equal(want["bgr"], g.input_op().data[:, [2, 1, 0]])
    assert np.array_equal(want["neg"], np.clip(-want["c1"].astype(np.int64), 0, 127))
    assert set(np.unique(want["mask"])) == {0, 127} and set(np.unique(want["hole"])) == {0, 127}
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.set_option("fuse_eltwise", fuse)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    m.close()
    check_through_files(g, g.input_op().data, want, tmp_path)
    g.ops[1].attrs["channel_order1"] = 3
    with pytest.raises(capi.TpuHipError, match="channel_order"):
        module().load(g)


def test_graph_with_dilate_and_reflection_pad(tmp_path):
    """a conv on a dilated map (what a transposed conv is lowered to) and one on a mirrored border"""
    b = graphs.Builder("dilate_reflect", graphs.BASE_SEED + 83, 2, (6, 12))
    x = b.input("input", 16, 9, 7)
    g = b.g
    n, c, h, w = g.by_name[x].shape
    g.add(graphs.Op("tpu.dilate", "holes", [x], (n, c, 2 * h - 1, 3 * w - 2), dict(ins0=2, ins1=1, fill_constant=-3)))
    cal = np.full((1, c, 2 * h - 1, 3 * w - 2), -3, np.int64)
    cal[:, :, ::2, ::3] = b.cal[x]
    b.cal["holes"] = cal
    g.add(graphs.Op("tpu.reflection_pad", "mirror", [x], (n, c, h, w + 5), dict(pads0=2, pads1=3)))
    b.cal["mirror"] = np.pad(b.cal[x], ((0, 0), (0, 0), (0, 0), (2, 3)), mode="reflect")
    c1 = b.conv("c1", "holes", 24, 3)
    c2 = b.conv("c2", "mirror", 24, 3)
    g.outputs = [c1, c2]
    want = oracle_graph.run(g)
    xin = g.input_op().data
    assert np.array_equal(want["mirror"], np.pad(xin, ((0, 0), (0, 0), (0, 0), (2, 3)), mode="reflect"))
    assert np.array_equal(want["holes"][:, :, ::2, ::3], xin) and (want["holes"][:, :, 1::2] == -3).all()
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.load(g)
    m.set_tensor("input", xin.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    m.close()
    check_through_files(g, xin, want, tmp_path)
    g.ops[2].attrs["pads1"] = w
    with pytest.raises(capi.TpuHipError, match="reflection_pad: pads"):
        mm = module()
        mm.load(g)
        mm.set_tensor("input", xin.astype(np.float32))
        mm.invoke()


def test_graph_with_reduce_ops_matches_the_oracle(tmp_path):
    """mean / max over the image, sum / min over the channels, with and without the reduced axes kept"""
    b = graphs.Builder("reduce_net", graphs.BASE_SEED + 83, 2, (6, 12))
    x = b.input("input", 8, 9, 7)
    c1 = b.conv("c1", x, 40, 3, relu=False)
    g = b.g
    f32 = lambda *v: np.array(v, np.float32)

    def red(t, name, shape, axes, rshift=None, mult=None):
        w = {} if rshift is None else dict(rshift=f32(rshift), multiplier=f32(mult))
        g.add(graphs.Op("tpu.reduce_" + t, name, [c1], shape, {"axes%d" % k: a for k, a in enumerate(axes)}, w,
                        "RSHIFT_AND_M_I8" if w else "NONE"))
        return name

    outs = [red("mean", "gmean", (2, 40, 1, 1), [2, 3], 9, 41), red("max", "gmax", (2, 40, 1, 1), [2, 3]),
            red("sum", "csum", (2, 1, 9, 7), [1], 6, 19), red("min", "cmin", (2, 9, 7), [1], 1, 3),
            red("max", "wmax", (2, 40, 9), [3], 0, 1), red("mean", "all", (2, 1), [1, 2, 3], 14, 90)]
    g.outputs = outs
    want = oracle_graph.run(g)
    for name in outs:
        assert len(np.unique(want[name])) > (3 if name == "all" else 8) or want[name].size < 4, name
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    m.close()
    check_through_files(g, g.input_op().data, want, tmp_path)
    # a sum without rescaling is no int8 tensor
    g.by_name["csum"].weights = {}
    m = module()
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    with pytest.raises(capi.TpuHipError, match="no int8 value"):
        m.invoke()
    m.close()


def test_graph_with_lrn_matches_the_oracle(tmp_path):
    """conv + ReLU -> LRN across channels -> max pool (the opening of GoogLeNet / AlexNet-style nets)"""
    rng = np.random.default_rng(8)
    b = graphs.Builder("lrn_net", graphs.BASE_SEED + 82, 2, (6, 12))
    x = b.input("input", 3, 20, 20)
    c1 = b.conv("c1", x, 48, 3, stride=2, relu=True)
    g = b.g
    shp = g.by_name[c1].shape
    idx = np.arange(256)
    sq = np.minimum(np.floor((idx / 16.0) ** 2 + 0.5), 255).astype(np.float32)
    pw = np.minimum(np.floor(255.0 * (1 + idx / 64.0) ** -0.75 + 0.5), 255).astype(np.float32)
    g.add(graphs.Op("tpu.lrn", "norm", [c1], shp,
                    dict(local_size=5, sum_rshift=4, lrn_rshift=8, quant_data0=13, quant_data1=2),
                    dict(sqr_lut=np.tile(sq, 32).reshape(1, 32, 16, 16), power_lut=np.tile(pw, 32).reshape(1, 32, 16, 16))))
    b.cal["norm"] = oracle_graph.run(g, upto="norm")["norm"][:1].astype(np.int64)
    p = b.pool_max("pool", "norm", 3, 2, (0, 1, 0, 1))
    g.outputs = [p]
    want = oracle_graph.run(g)
    assert len(np.unique(want["norm"])) > 8 and (want["norm"] != want["c1"]).mean() > 0.3
    m = module()
    m.set_option("keep_all_tensors", 1)
    m.load(g)
    m.set_tensor("input", g.input_op().data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        assert np.array_equal(m.get_tensor_i8(op.name), want[op.name].reshape(op.shape)), op.name
    m.close()
    check_through_files(g, g.input_op().data, want, tmp_path)
    g.by_name["norm"].weights["sqr_lut"] = g.by_name["norm"].weights["sqr_lut"] + 0.5
    with pytest.raises(capi.TpuHipError, match="not an integer"):
        module().load(g)


def test_graph_with_uint8_input_and_scale_lut_matches_the_oracle(tmp_path):
    """uint8 image -> ScaleLut (per-channel 256-entry tables) -> conv"""
    rng = np.random.default_rng(6)
    b = graphs.Builder("scale_lut", graphs.BASE_SEED + 80, 2, (6, 12))
    x8 = b.input("x8", 3, 20, 18)                # calibrates the conv; replaced below
    c1 = b.conv("c1", x8, 24, 3, relu=True)
    g = b.g
    shape = g.by_name["x8"].shape
    img = rng.integers(0, 256, shape).astype(np.uint8)
    img.flat[:4] = [0, 127, 128, 255]
    idx = np.arange(256)
    scale, bias = np.array([0.9, 1.0, 0.4]), np.array([-110.0, -128.0, 11.0])
    table = np.clip(np.floor(idx[None] * scale[:, None] + bias[:, None] + 0.5), -128, 127)
    fin = graphs.Op("tpu.input", "input", [], shape)
    fin.quant = "UINT8"
    fin.data = img
    sl = graphs.Op("tpu.scale_lut", "x8", ["input"], shape, {},
                   dict(table=table.astype(np.float32).reshape(-1)))
    g.ops[0:1] = [fin, sl]
    g.by_name["input"] = fin
    g.by_name["x8"] = sl
    g.outputs = [c1]
    want = oracle_graph.run(g)
    assert np.array_equal(want["x8"][:, 1], (img[:, 1].astype(np.int16) - 128).astype(np.int8))
    m = module()
    m.load(g)
    m.set_tensor("input", img.astype(np.float32))
    m.invoke()
    assert np.array_equal(m.get_tensor("input"), img.astype(np.float32))
    for name in ("x8", c1):
        assert np.array_equal(m.get_tensor_i8(name), want[name]), name
    assert len(np.unique(want[c1])) > 8
    with pytest.raises(capi.TpuHipError, match="not a uint8 value"):
        m.set_tensor("input", img.astype(np.float32) - 1.0)
    m.close()
    check_through_files(g, img, want, tmp_path)
    # a signed tensor in front of a ScaleLut, and a UINT8 tensor in front of anything else, are refused
    g2 = graphs.Graph("bad", 1)
    g2.add(graphs.Op("tpu.input", "input", [], (1, 3, 4, 4))).data = np.zeros((1, 3, 4, 4), np.int8)
    g2.add(graphs.Op("tpu.scale_lut", "s", ["input"], (1, 3, 4, 4), {},
                     dict(table=np.zeros(768, np.float32))))
    with pytest.raises(capi.TpuHipError, match="UINT8 tensor"):
        module().load(g2)
    g3 = graphs.Graph("bad", 1)
    i3 = g3.add(graphs.Op("tpu.input", "input", [], (1, 16, 4, 4)))
    i3.quant = "UINT8"
    i3.data = np.zeros((1, 16, 4, 4), np.uint8)
    g3.add(graphs.Op("tpu.relu", "r", ["input"], (1, 16, 4, 4)))
    with pytest.raises(capi.TpuHipError, match="only read by ScaleLut"):
        module().load(g3)


@pytest.mark.parametrize("cfg", [
    # ic, ih, iw, oc, k, stride, pads(t,b,l,r), dil, groups, out_hw
    (24, 7, 6, 40, 3, (2, 2), (1, 1, 1, 1), (1, 1), 1, (14, 12)),     # output_padding 1
    (16, 5, 9, 24, 4, (2, 3), (1, 1, 2, 2), (1, 1), 2, (10, 24)),
    (20, 6, 6, 20, 3, (1, 1), (0, 0, 0, 0), (2, 2), 20, (10, 10)),    # depthwise, dilated
    (12, 8, 5, 18, 2, (2, 2), (0, 0, 0, 0), (1, 1), 1, (16, 10)),     # the 2x upsampling deconv
])
def test_deconv_graph_matches_the_oracle(cfg):
    ic, ih, iw, oc, k, stride, pads, dil, grp, out_hw = cfg
    rng = np.random.default_rng(ic + oc + k)
    g = graphs.Graph("deconv", 1)
    x = rng.integers(-128, 128, (2, ic, ih, iw)).astype(np.int8)
    inp = g.add(graphs.Op("tpu.input", "input", [], x.shape))
    inp.data = x
    w = np.clip(np.rint(rng.normal(0, 30, (oc, ic // grp, k, k))), -127, 127).astype(np.float32)
    bias = rng.integers(-2000, 2000, oc).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
    rsh = rng.integers(5, 12, oc).astype(np.float32)
    g.add(graphs.Op("tpu.deconv_2d", "up", ["input"], (2, oc) + out_hw,
                    dict(kernel_h=k, kernel_w=k, stride_h=stride[0], stride_w=stride[1],
                         padding_t=pads[0], padding_b=pads[1], padding_l=pads[2], padding_r=pads[3],
                         dilation_h=dil[0], dilation_w=dil[1], group=grp, with_bias=1, do_relu=1),
                    dict(filter=w.ravel(), bias=bias, rshift=rsh, multiplier=mult), "RSHIFT_AND_M_I32"))
    g.outputs = ["up"]
    want = oracle_graph.run(g)
    m = module()
    m.load(g)
    m.set_tensor("input", x.astype(np.float32))
    m.invoke()
    assert np.array_equal(m.get_tensor_i8("up"), want["up"])
    assert len(np.unique(want["up"])) > 8
    m.close()


def test_graph_with_fp32_edges_quantizes_and_dequantizes_like_the_oracle(tmp_path):
    """fp32 input -> QuantOp -> conv -> conv -> QuantOp -> fp32 output"""
    rng = np.random.default_rng(5)
    b = graphs.Builder("edges", graphs.BASE_SEED + 79, 3, (6, 12))
    x8 = b.input("x8", 20, 9, 7)                 # calibrates the convs; replaced by the quant op below
    c1 = b.conv("c1", x8, 32, 3, relu=True)
    c2 = b.conv("c2", c1, 24, 1, relu=False)
    g = b.g
    # put an fp32 input and a QuantOp in front, a dequantising QuantOp behind
    shape = g.by_name["x8"].shape
    xf = rng.normal(0, 1.2, shape).astype(np.float32)
    xf.flat[:8] = [0.5 / 31.75, -0.5 / 31.75, 1.5 / 31.75, 4.1, -4.1, 100.0, -100.0, 0.0]
    fin = graphs.Op("tpu.input", "input", [], shape)
    fin.quant = "NONE"
    fin.data = xf
    q = graphs.Op("tpu.quant", "x8", ["input"], shape, dict(scale=31.75))
    old = g.ops[0]
    g.ops[0:1] = [fin, q]
    g.by_name["input"] = fin
    g.by_name["x8"] = q
    dq = graphs.Op("tpu.quant", "out", [c2], g.by_name[c2].shape, dict(scale=0.0207))
    dq.quant = "NONE"
    g.add(dq)
    g.outputs = ["out"]
    want = oracle_graph.run(g)
    assert want["out"].dtype == np.float32 and want["x8"].dtype == np.int8
    m = module()
    m.load(g)
    m.set_tensor("input", xf)
    m.invoke()
    assert np.array_equal(m.get_tensor("input"), xf)
    for name in ("x8", c1, c2):
        assert np.array_equal(m.get_tensor_i8(name), want[name]), name
    got = m.get_tensor("out")
    assert got.dtype == np.float32 and np.array_equal(got, want["out"])
    assert len(np.unique(got)) > 8
    with pytest.raises(capi.TpuHipError, match="fp32"):
        m.get_tensor_i8("out")
    m.close()
    check_through_files(g, xf, want, tmp_path)
    # an INT8 op fed with fp32 data is refused
    g2 = graphs.Graph("bad", 1)
    i2 = g2.add(graphs.Op("tpu.input", "input", [], (1, 16, 4, 4)))
    i2.quant = "NONE"
    i2.data = np.zeros((1, 16, 4, 4), np.float32)
    g2.add(graphs.Op("tpu.relu", "r", ["input"], (1, 16, 4, 4)))
    with pytest.raises(capi.TpuHipError, match="QuantOp in front"):
        module().load(g2)


def test_fp32_network_quantized_with_the_host_helpers_tracks_the_fp32_result(tmp_path):
    """an fp32 network (torch) + max-abs calibration thresholds -> INT8 operands from the
    quantisation helpers -> the GPU graph.  Bit-exact against the oracle as always, and close to
    the fp32 network layer by layer, which is what those helpers are for."""
    import torch
    import torch.nn.functional as F
    from tpu_compiler_amd import quantize as Q
    torch.manual_seed(3)
    rng = np.random.default_rng(3)
    n, hw = 4, 20
    x = torch.tensor(rng.normal(0, 1, (n, 3, hw, hw)).astype(np.float32)).clamp(-3, 3)
    w1, b1 = torch.randn(16, 3, 3, 3) * 0.3, torch.randn(16) * 0.2
    w2, b2 = torch.randn(16, 16, 3, 3) * 0.1, torch.randn(16) * 0.2
    w3, b3 = torch.randn(24, 16, 1, 1) * 0.3, torch.randn(24) * 0.1
    wf, bf = torch.randn(10, 24) * 0.4, torch.randn(10) * 0.1
    a1 = F.relu(F.conv2d(x, w1, b1, padding=1))
    a2 = F.conv2d(a1, w2, b2, padding=1)
    a3 = F.relu(a1 + a2)
    a4 = F.conv2d(a3, w3, b3)
    a5 = F.leaky_relu(a4, 0.1)
    a6 = a5.mean(dim=(2, 3), keepdim=True)
    a7 = F.linear(a6.flatten(1), wf, bf)
    acts = dict(input=x, c1=a1, c2=a2, add=a3, c3=a4, leaky=a5, gap=a6, fc=a7)
    thr = {k: float(v.abs().max()) for k, v in acts.items()}

    g = graphs.Graph("quantized", 0)
    xin = g.add(graphs.Op("tpu.input", "input", [], (n, 3, hw, hw)))
    xin.data = np.clip(np.floor(x.numpy() * (127.0 / thr["input"]) + 0.5), -128, 127).astype(np.int8)

    def conv(name, src, w, b, tx, ty, k, pad, relu):
        wq, bq, rs, mu = Q.quantize_conv(w.numpy(), b.numpy(), tx, ty)
        oc = w.shape[0]
        g.add(graphs.Op("tpu.conv_2d", name, [src], (n, oc, hw, hw),
                        dict(kernel_h=k, kernel_w=k, stride_h=1, stride_w=1, dilation_h=1, dilation_w=1,
                             padding_t=pad, padding_b=pad, padding_l=pad, padding_r=pad, group=1, do_relu=int(relu),
                             with_bias=1),
                        dict(filter=wq, bias=bq, rshift=rs, multiplier=mu), "RSHIFT_AND_M_I32"))

    conv("c1", "input", w1, b1, thr["input"], thr["c1"], 3, 1, True)
    conv("c2", "c1", w2, b2, thr["c1"], thr["c2"], 3, 1, False)
    rs, mu = Q.quantize_rescale([thr["c1"], thr["c2"]], thr["add"])
    g.add(graphs.Op("tpu.eltwise_add", "add", ["c1", "c2"], (n, 16, hw, hw), dict(do_relu=1),
                    dict(rshift=rs, multiplier=mu), "RSHIFT_AND_M_I8"))
    conv("c3", "add", w3, b3, thr["add"], thr["c3"], 1, 0, False)
    g.add(graphs.Op("tpu.leaky_relu", "leaky", ["c3"], (n, 24, hw, hw), dict(negative_slope=0.1),
                    Q.quantize_leaky_relu(0.1, thr["c3"], thr["leaky"]), "RSHIFT_AND_M_I8"))
    rs, mu = Q.quantize_rescale([thr["leaky"]], thr["gap"], divisor=hw * hw)
    g.add(graphs.Op("tpu.pool_avg_2d", "gap", ["leaky"], (n, 24, 1, 1),
                    dict(kernel_h=hw, kernel_w=hw, stride_h=1, stride_w=1, padding_t=0, padding_b=0, padding_l=0,
                         padding_r=0, do_relu=0, count_include_pad=1, pad_value=0),
                    dict(rshift=rs, multiplier=mu), "RSHIFT_AND_M_I8"))
    g.add(graphs.Op("tpu.reshape", "flat", ["gap"], (n, 24)))
    wq, bq, rs, mu = Q.quantize_fc(wf.numpy(), bf.numpy(), thr["gap"], thr["fc"])
    g.add(graphs.Op("tpu.fully_connected", "fc", ["flat"], (n, 10), dict(do_relu=0),
                    dict(filter=wq, bias=bq, rshift=rs, multiplier=mu), "RSHIFT_AND_M_I32"))
    g.outputs = ["fc"]

    want = oracle_graph.run(g)
    m = module()
    m.load(g)
    m.set_tensor("input", xin.data.astype(np.float32))
    m.invoke()
    for op in g.ops:
        got = m.get_tensor_i8(op.name)
        assert np.array_equal(got, want[op.name].reshape(op.shape)), op.name
        if op.name in acts and op.name != "input":
            ref = acts[op.name].numpy().reshape(op.shape)
            deq = got.astype(np.float64) * thr[op.name] / 127.0
            cos = (deq * ref).sum() / np.sqrt((deq * deq).sum() * (ref * ref).sum())
            assert cos > 0.995, (op.name, cos)
            assert np.abs(deq - ref).max() < 0.06 * thr[op.name], (op.name, np.abs(deq - ref).max() / thr[op.name])
    m.close()
    check_through_files(g, xin.data, want, tmp_path)


def _random_graph(it):
    """a random DAG of convs (1x1 / 3x3 / depthwise, some strided), adds, leaky relu, clip, max pool,
    upsample and concat over earlier tensors; None when the builder's guards reject it"""
    rng = np.random.default_rng(424200 + it)
    b = graphs.Builder("fz%d" % it, graphs.BASE_SEED + 1000 + it, int(rng.integers(1, 3)), (5, 11))
    hw = int(rng.integers(5, 15))
    vals = [b.input("input", int(rng.choice([3, 16, 24, 64])), hw, hw + int(rng.integers(0, 4)))]
    g = b.g
    kinds = ["conv1", "conv3", "add", "leaky", "clip", "pool", "concat", "conv1", "conv3", "add", "up", "dw"]
    try:
        for k in range(int(rng.integers(3, 14))):
            kind = kinds[int(rng.integers(0, 12))]
            src = vals[int(rng.integers(0, len(vals)))] if rng.integers(0, 3) else vals[-1]
            shp = g.by_name[src].shape
            name = "%s_%d" % (kind, k)
            if kind == "conv1":
                s = 2 if (rng.integers(0, 4) == 0 and shp[2] > 3) else 1
                vals.append(b.conv(name, src, int(rng.choice([16, 24, 64, 128, 40])), 1, stride=s,
                                   relu=bool(rng.integers(0, 2))))
            elif kind == "conv3":
                vals.append(b.conv(name, src, int(rng.choice([16, 24, 64, 72])), 3, relu=bool(rng.integers(0, 2))))
            elif kind == "dw":
                if shp[1] >= 8:
                    vals.append(b.conv(name, src, shp[1], 3, groups=shp[1], relu=bool(rng.integers(0, 2))))
            elif kind == "add":
                same = [v for v in vals if g.by_name[v].shape == shp and v != "input"]
                if same and src != "input":
                    other = same[int(rng.integers(0, len(same)))]
                    vals.append(b.add(name, [src, other] if rng.integers(0, 2) else [other, src],
                                      bool(rng.integers(0, 2))))
            elif kind == "leaky":
                vals.append(b.leaky(name, src))
            elif kind == "clip":
                vals.append(b.clip(name, src, -int(rng.integers(0, 100)), int(rng.integers(1, 100))))
            elif kind == "pool":
                if shp[2] >= 3 and shp[3] >= 3:
                    vals.append(b.pool_max(name, src, 2, 2, (0, 0, 0, 0)))
            elif kind == "up":
                if shp[2] * shp[3] <= 400:
                    vals.append(b.upsample(name, src, 2))
            else:
                same = [v for v in vals if g.by_name[v].shape[0] == shp[0] and g.by_name[v].shape[2:] == shp[2:]]
                if len(same) >= 2:
                    take = rng.choice(len(same), size=min(len(same), int(rng.integers(2, 4))), replace=False)
                    vals.append(b.concat(name, [same[int(i)] for i in take]))
    except (AssertionError, ValueError):
        return None
    if len(vals) < 2:
        return None
    return b.finish(vals[1:][-3:])


def test_random_graphs_with_and_without_fusion_and_pairing():
    """80 random graphs: whatever the interpreter folds into conv epilogues, packs into one launch
    or leaves unwritten, every tensor it keeps must equal the oracle's"""
    ran = fused = 0
    for it in range(80):
        g = _random_graph(it)
        if g is None:
            continue
        want = oracle_graph.run(g)
        for fuse, pair, keep in ((1, 1, 1), (1, 1, 0), (0, 0, 1)):
            m = module()
            m.set_option("keep_all_tensors", keep)
            m.set_option("fuse_eltwise", fuse)
            m.set_option("pair_convs", pair)
            m.load(g)
            m.set_tensor("input", g.input_op().data.astype(np.float32))
            m.invoke()
            for name in ([op.name for op in g.ops] if keep else g.outputs):
                assert np.array_equal(m.get_tensor_i8(name), want[name].reshape(g.by_name[name].shape)), \
                    (it, fuse, pair, keep, name, [(o.type, o.name, o.inputs) for o in g.ops])
            m.close()
        ran += 1
        fused += any(o.type == "tpu.eltwise_add" for o in g.ops)
    assert ran >= 60 and fused >= 20, (ran, fused)


def _random_single_op_graph(it):
    """one transposed conv (dense / grouped / depthwise, strides, dilation, pads, output padding),
    one reduce (kind, consecutive axes, kept or dropped, rescaled or not) or one FC behind an input"""
    f32 = lambda *v: np.array(v, np.float32)
    rng = np.random.default_rng(616100 + it)
    kind = ["deconv", "reduce", "fc"][int(rng.integers(0, 3))]
    g = graphs.Graph("fz", 1)
    n = int(rng.integers(1, 3))
    if kind == "deconv":
        grp = int(rng.choice([1, 1, 2, 0]))
        ic = int(rng.integers(1, 40))
        oc = int(rng.integers(1, 40))
        if grp == 0:
            grp = ic
            oc = ic
        elif grp == 2:
            (ic, oc) = (2 * int(rng.integers(1, 16)), 2 * int(rng.integers(1, 16)))
        (ih, iw) = (int(rng.integers(1, 10)), int(rng.integers(1, 10)))
        k = int(rng.integers(1, 5))
        stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pads = tuple((int(min(v, dil[i // 2] * (k - 1))) for (i, v) in enumerate(rng.integers(0, 3, 4))))
        oh = (ih - 1) * stride[0] - pads[0] - pads[1] + dil[0] * (k - 1) + 1 + int(rng.integers(0, stride[0]))
        ow = (iw - 1) * stride[1] - pads[2] - pads[3] + dil[1] * (k - 1) + 1 + int(rng.integers(0, stride[1]))
        if oh < 1 or ow < 1:
            return (None, kind)
        x = rng.integers(-128, 128, (n, ic, ih, iw)).astype(np.int8)
        g.add(graphs.Op("tpu.input", "input", [], x.shape)).data = x
        w = np.clip(np.rint(rng.normal(0, 30, (oc, ic // grp, k, k))), -127, 127).astype(np.float32)
        bias = rng.integers(-2000, 2000, oc).astype(np.float32)
        mult = (rng.integers(1 << 23, 1 << 24, oc) * 128).astype(np.float32)
        rsh = rng.integers(3, 11, oc).astype(np.float32)
        g.add(graphs.Op("tpu.deconv_2d", "y", ["input"], (n, oc, oh, ow),
                        dict(kernel_h=k, kernel_w=k, stride_h=stride[0], stride_w=stride[1], padding_t=pads[0],
                             padding_b=pads[1], padding_l=pads[2], padding_r=pads[3], dilation_h=dil[0],
                             dilation_w=dil[1], group=grp, with_bias=1, do_relu=int(rng.integers(0, 2))),
                        dict(filter=w.ravel(), bias=bias, rshift=rsh, multiplier=mult), "RSHIFT_AND_M_I32"))
    elif kind == "reduce":
        (c, ih, iw) = (int(rng.integers(1, 60)), int(rng.integers(1, 12)), int(rng.integers(1, 12)))
        x = rng.integers(-128, 128, (n, c, ih, iw)).astype(np.int8)
        g.add(graphs.Op("tpu.input", "input", [], x.shape)).data = x
        t = ["mean", "sum", "max", "min"][int(rng.integers(0, 4))]
        a0 = int(rng.integers(1, 4))
        a1 = int(rng.integers(a0, 4))
        axes = list(range(a0, a1 + 1))
        keep = bool(rng.integers(0, 2))
        full = [n, c, ih, iw]
        shape = tuple(1 if i in axes else d for i, d in enumerate(full)) if keep else \
            tuple(d for i, d in enumerate(full) if i not in axes)
        cnt = int(np.prod([full[i] for i in axes]))
        if t in ("mean", "sum") or rng.integers(0, 2):
            rs = int(rng.integers(0, 15))
            m_ = int(rng.integers(1, 256))
            wts = dict(rshift=f32(rs), multiplier=f32(m_))
            pt = "RSHIFT_AND_M_I8"
        else:
            wts = {}
            pt = "NONE"
        g.add(graphs.Op("tpu.reduce_" + t, "y", ["input"], shape, {"axes%d" % k: a for k, a in enumerate(axes)},
                        wts, pt))
    else:
        (m_, k, nn) = (n, int(rng.integers(1, 600)), int(rng.integers(1, 300)))
        x = rng.integers(-128, 128, (m_, k, 1, 1)).astype(np.int8)
        g.add(graphs.Op("tpu.input", "input", [], x.shape)).data = x
        sig = min(30.0, 900.0 / k ** 0.5)
        w = np.clip(np.rint(rng.normal(0, sig, (nn, k))), -127, 127).astype(np.float32)
        bias = rng.integers(-2000, 2000, nn).astype(np.float32)
        mult = f32(float(int(rng.integers(1 << 23, 1 << 24)) * 128))
        g.add(graphs.Op("tpu.fully_connected", "y", ["input"], (m_, nn), dict(do_relu=int(rng.integers(0, 2))),
                        dict(filter=w, bias=bias, rshift=f32(int(rng.integers(4, 12))), multiplier=mult),
                        "RSHIFT_AND_M_I32"))
    g.outputs = ["y"]
    return (g, kind)


@pytest.mark.parametrize("x_shape,w_shape,y_shape,lt,ot", [
    ((4, 3, 28), (4, 5, 28), (4, 3, 5), 0, 0),          # the batched form of TPUOperationSupport.cpp:566
    ((4, 3, 28), (5, 28), (4, 3, 5), 0, 0),             # :567: one matmul with m = 12
    ((2, 8, 3, 48), (6, 20, 48), (2, 3, 8, 20), 1, 0),  # input_transpose
    ((2, 3, 8, 48), (6, 20, 48), (2, 8, 3, 20), 0, 1),  # output_transpose
    ((2, 8, 3, 48), (2, 3, 20, 48), (2, 8, 3, 20), 1, 1),
])
def test_fully_connected_batched_and_transposed_graphs(x_shape, w_shape, y_shape, lt, ot):
    """FullyConnectedOpKernel with a batch and with either transpose (core/fullyconnected.cpp:52-88),
    through the module interpreter, against the oracle's restatement"""
    rng = np.random.default_rng(sum(x_shape) + 10 * lt + 20 * ot)
    f32 = lambda v: np.asarray(v, np.float32).reshape(-1)
    g = graphs.Graph("fc_batched", 77)
    x = rng.integers(-128, 128, x_shape).astype(np.int8)
    g.add(graphs.Op("tpu.input", "input", [], x.shape)).data = x
    batch = int(np.prod(w_shape[:-2]))
    w = np.clip(np.rint(rng.normal(0, 25, w_shape)), -127, 127).astype(np.float32)
    bias = rng.integers(-2000, 2000, (batch, w_shape[-2])).astype(np.float32)
    mult = (rng.integers(1 << 23, 1 << 24, batch) * 128).astype(np.float32)
    rsh = rng.integers(6, 11, batch).astype(np.float32)
    g.add(graphs.Op("tpu.fully_connected", "y", ["input"], y_shape,
                    dict(do_relu=1, input_transpose=lt, output_transpose=ot),
                    dict(filter=w, bias=bias, rshift=rsh, multiplier=mult), "RSHIFT_AND_M_I32"))
    g.outputs = ["y"]
    want = oracle_graph.run(g)["y"]
    m = module()
    m.load(g)
    m.set_tensor("input", x.astype(np.float32))
    m.invoke()
    got = m.get_tensor_i8("y")
    assert dict(m.kernels())["y"] == "fc/batched"
    assert np.array_equal(got.reshape(y_shape), want.reshape(y_shape))
    assert len(np.unique(want)) > 8
    m.close()


def test_random_deconv_reduce_and_fc_graphs():
    ran = {}
    for it in range(240):
        g, kind = _random_single_op_graph(it)
        if g is None:
            continue
        want = oracle_graph.run(g)["y"]
        m = module()
        m.load(g)
        m.set_tensor("input", g.input_op().data.astype(np.float32))
        m.invoke()
        got = m.get_tensor_i8("y")
        assert np.array_equal(got, want.reshape(got.shape)), (it, [(o.type, o.shape, o.attrs) for o in g.ops])
        m.close()
        ran[kind] = ran.get(kind, 0) + 1
    assert len(ran) == 3 and min(ran.values()) > 50, ran
