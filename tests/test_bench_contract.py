"""The benchmark's command-line contract: what can be checked without a GPU (the refusal of
more than one GPU, the recorded tile file, the CPU baseline leg) and, on the GPU, the one JSON
line with its required keys."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_recorded_tiles_name_layers_and_variants_that_exist():
    sys.path.insert(0, ROOT)
    import bench
    from tpu_compiler_amd import capi, graphs
    lib = capi.bind()
    names = []
    while lib.tpuhip_conv2d_tile_name(len(names)):
        names.append(lib.tpuhip_conv2d_tile_name(len(names)).decode())
    # a layer that opens a launch of two chained convs is recorded under that kernel's name
    n_chain = 0
    while lib.tpuhip_conv2d_chain_variant_name(n_chain):
        names.append(lib.tpuhip_conv2d_chain_variant_name(n_chain).decode())
        n_chain += 1
    for cfg, rel in bench.RECORDED_TILES.items():
        tiles = json.load(open(os.path.join(ROOT, rel)))
        g = graphs.CONFIGS[cfg]()
        convs = {o.name for o in g.ops if o.type == "tpu.conv_2d"}
        assert set(tiles) <= convs, sorted(set(tiles) - convs)
        assert set(tiles.values()) <= set(names), sorted(set(tiles.values()) - set(names))
        assert len(tiles) >= {"cfg3": 40, "cfg4": 30, "cfg5": 60}[cfg]      # every MFMA conv of the graph


def test_committed_traffic_figures_name_kernel_variants_the_library_still_has():
    """bench.py takes roofline.traffic from profiles/resnet50_b32_bench_traffic.json by kernel variant name:
    a variant renamed or removed in the library must not leave a stale entry behind"""
    from tpu_compiler_amd import capi
    lib = capi.bind()
    names = set()
    i = 0
    while lib.tpuhip_conv2d_tile_name(i):
        names.add(lib.tpuhip_conv2d_tile_name(i).decode())
        i += 1
    i = 0
    while lib.tpuhip_conv2d_chain_variant_name(i):
        names.add(lib.tpuhip_conv2d_chain_variant_name(i).decode())
        i += 1
    t = json.load(open(os.path.join(ROOT, "profiles", "resnet50_b32_bench_traffic.json")))
    assert t["kernels"] and set(t["kernels"]) <= names, sorted(set(t["kernels"]) - names)
    for k, v in t["kernels"].items():
        assert v["fetch_KiB"] > 0 and v["write_KiB"] > 0, k


def test_cpu_baseline_leg_reports_what_it_ran():
    sys.path.insert(0, ROOT)
    import bench
    from tpu_compiler_amd import graphs
    out = bench.cpu_baseline(graphs.CONFIGS["cfg1"], 2, seconds=0.2)
    assert out["kind"] == "port" and out["unit"] == "images/s" and out["value"] > 0
    assert out["cores"] >= 1 and "cfg1" in out["sample"] and "2 images" in out["sample"]


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_contract_keys():
    r = subprocess.run([sys.executable, BENCH, "--config", "cfg2", "--steps", "5", "--warmup", "2", "--host-io"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert d["metric"] == "images_per_sec" and d["unit"] == "images/s" and d["higher_is_better"] is True
    assert "workload" in d["config"] and "model" not in d["config"]
    assert np.isclose(d["value"], d["config"]["global_batch"] / (d["ms_per_step"] / 1e3), rtol=1e-2)
    r_ = d["roofline"]
    assert r_["bound"] in ("hbm", "mfma") and np.isclose(r_["frac"], r_["achieved"] / r_["peak"], atol=1e-3)
    f = d["graph_floor"]
    assert f["launches"] >= 2 and np.isclose(f["floor_ms"], f["data_ms"] + f["launch_ms"], atol=2e-4)
    assert f["step_over_floor"] >= 1.0 and r_["against_hbm"]["lower_roof"] in ("hbm", "mfma")
    # the leg with host buffers in and out every step is reported beside the value, and is slower
    assert d["host_io"]["ms_per_step"] > d["ms_per_step"] and d["host_io"]["host_bytes_in"] > 0
    c = d["cpu_baseline"]
    assert c["kind"] in ("port", "reference") and c["value"] > 0 and c["cores"] >= 1 and c["sample"]


def test_activation_statistics_of_the_parity_object():
    sys.path.insert(0, ROOT)
    import numpy as np
    import bench

    class Op:
        def __init__(self, name):
            self.name = name
    a = np.array([0, 0, 127, -128, 5, -5, 1, 2], np.int8)
    b = np.zeros(8, np.float32)                      # an fp32 edge tensor: not counted
    s = bench.activation_stats([Op("a"), Op("b"), Op("missing")], {"a": a, "b": b}, {"a": 1000, "x": 77})
    assert s == {"int8_elements": 8, "zero_frac": 0.25, "saturated_frac": 0.25, "fp32_guard_max": 1000}
    assert bench.activation_stats([Op("b")], {"b": b}, {}) is None



def test_op_bench_describes_itself_without_a_gpu():
    r = subprocess.run([sys.executable, "-m", "tpu_compiler_amd.op_bench", "--help"], capture_output=True, text=True,
                       timeout=120, cwd=ROOT)
    assert r.returncode == 0 and "--iters" in r.stdout


@pytest.mark.gpu
def test_op_bench_prints_a_row_per_op():
    r = subprocess.run([sys.executable, "-m", "tpu_compiler_amd.op_bench", "--iters", "3"], capture_output=True,
                       text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    rows = [l for l in r.stdout.splitlines() if " TB/s " in l]
    assert len(rows) == 14
    for l in rows:
        us = float(l.split(" us (host")[0].split()[-1])
        assert 1.0 < us < 1000.0, l
