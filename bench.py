#!/usr/bin/env python3
"""Benchmark of the INT8 interpreter path on one MI355X.

A step is one pass of the whole quantized graph over one batch of synthetic
input already resident in HBM.  Default workload: the ResNet-50-shaped INT8
graph at batch 32.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg3]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense INT8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s
LAUNCH_FLOOR_US = 2.4     # an empty kernel behind another on one stream, measured (profiles/machine_ceilings.txt)
# conv tile variant per layer as an earlier run of this benchmark chose them by timing: used
# by default so that runs, and the committed profile of this command, execute the same kernels
RECORDED_TILES = {"cfg3": os.path.join("tpu_compiler_amd", "tiles", "cfg3_b32.json"),
                  "cfg4": os.path.join("tpu_compiler_amd", "tiles", "cfg4_b64.json"),
                  "cfg5": os.path.join("tpu_compiler_amd", "tiles", "cfg5_b8.json")}


def conv_bytes(op, graph, fused_add=None, stored=True):
    """algorithmic bytes of a conv / fc launch: int8 input + output + filter, 12 B of int32
    parameters per output channel; with an eltwise add folded into the epilogue also the add's
    other operand and its sum; without the conv result itself where that is not written"""
    import numpy as np
    x = graph.by_name[op.inputs[0]].shape
    oc = op.shape[1]
    n = int(np.prod(x)) + int(op.weights["filter"].size) + 12 * oc
    if stored:
        n += int(np.prod(op.shape))
    if fused_add is not None:
        n += 2 * int(np.prod(fused_add.shape))
    return n


def host_cpu():
    """model name, physical cores and logical CPUs of this host (from /proc/cpuinfo)"""
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            k, _, v = line.partition(":")
            k, v = k.strip(), v.strip()
            if k == "model name":
                model = v
            elif k == "physical id":
                phys = v
            elif k == "core id":
                core = v
            elif not k and phys is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    return {"model": model, "physical_cores": len(cores) or None, "logical_cpus": os.cpu_count()}


def _set_threads(n):
    """OpenMP threads of the oracle library and of PyTorch's CPU ops"""
    import ctypes
    import torch
    torch.set_num_threads(n)
    try:
        ctypes.CDLL("libgomp.so.1").omp_set_num_threads(n)
    except OSError:
        pass


def _timed(fn, seconds, max_passes=20):
    fn()                                     # page in
    passes, t0 = 0, time.perf_counter()
    while passes < max_passes and (passes == 0 or time.perf_counter() - t0 < seconds):
        fn()
        passes += 1
    return passes, time.perf_counter() - t0


def activation_stats(ops, tensors, guards):
    """What the parity check ran on: share of zero and of saturated (-128 / 127) bytes over every int8
    tensor of the graph as the oracle computed it, and the largest fp32-exactness guard of a conv / fc
    output (sum |a * w| + |bias|, which has to stay below 2^24 for the reference's fp32 sums to be exact)."""
    import numpy as np
    total = zeros = saturated = 0
    for op in ops:
        a = tensors.get(op.name)
        if a is None or a.dtype != np.int8:
            continue
        total += a.size
        zeros += int(np.count_nonzero(a == 0))
        saturated += int(np.count_nonzero((a == 127) | (a == -128)))
    if not total:
        return None
    return {"int8_elements": total, "zero_frac": round(zeros / total, 4), "saturated_frac": round(saturated / total, 4),
            "fp32_guard_max": int(max(guards.values())) if guards else None}


def cpu_baseline(graph_fn, images, seconds=12.0, legs=("dataflow_4thr", "dataflow_all", "oracle_all"),
                 keep_results=None):
    """CPU restatements of the reference on a bounded sample of the same workload, on this host:
    dataflow_*: the reference's data flow -- float-stored NCHW tensors, fp32 conv / inner product /
    pooling through oneDNN (PyTorch CPU ops), float and integer epilogues, the graph run as an N=1
    graph once per image (MlirModuleInterpreter.cpp:383-405) -- at the 4 threads the reference's
    regression pins (regression/run_regression.sh:14) and at all CPUs; oracle_all: the integer-exact
    C/OpenMP oracle.  The top-level value is the data-flow leg at all CPUs."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_dataflow
    import oracle_graph
    g = graph_fn(batch=images)
    all_cpus = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    per_leg = max(0.1, seconds / max(1, len(legs)))
    out_legs = {}
    for leg in legs:
        threads = 4 if leg.endswith("_4thr") else all_cpus
        _set_threads(threads)
        if leg.startswith("dataflow"):
            n_img = max(1, min(images, 4))
            passes, dt = _timed(lambda: oracle_dataflow.run(g, keep=g.outputs, images=n_img), per_leg)
            done = passes * n_img
            what = "%d N=1 passes (%.1f s) of the fp32 data-flow restatement" % (done, dt)
        else:
            passes, dt = _timed(lambda: oracle_graph.run(g, keep=g.outputs), per_leg)
            done = passes * images
            what = "%d passes of a batch of %d images (%.1f s) through the integer-exact C/OpenMP oracle" % (
                passes, images, dt)
        out_legs[leg] = {"value": round(done / dt, 2), "unit": "images/s", "cores": threads, "what": what}
    _set_threads(all_cpus)
    if keep_results is not None:
        keep_results.update(oracle_graph.run(g, guards=keep_results.setdefault("__guards__", {})))
    head = out_legs.get("dataflow_all") or next(iter(out_legs.values()))
    return {"value": head["value"], "unit": "images/s", "cores": head["cores"], "kind": "port",
            "sample": "%s, %d images: %s" % (g.name, images, head["what"]),
            "host": host_cpu(), "legs": out_legs}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # 200 steps: with 50 the wall-clock figure of a 0.6 ms step still moves by 2 % from run to run
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"])
    ap.add_argument("--batch", type=int, default=0,
                    help="images per step instead of the configuration's own batch (a different workload: "
                         "named as such in config.workload, recorded tiles not applied)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--host-io", action="store_true",
                    help="also time steps that take the input from and return the outputs to host fp32 "
                         "buffers (set_tensor + invoke + get_tensor), reported as host_io, never as value")
    ap.add_argument("--per-layer", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--save-tiles", default="", help="write the conv tile chosen for every layer")
    ap.add_argument("--tiles", default="", help="use the conv tiles recorded in this file instead "
                                                "of timing the variants (repeatable profiling); "
                                                "default for cfg3 / cfg4 / cfg5: the files under tpu_compiler_amd/tiles")
    ap.add_argument("--autotune", action="store_true",
                    help="time the conv tile variants on first use even where a recorded choice exists")
    ap.add_argument("--keep-all", action="store_true",
                    help="write every tensor of the graph (the reference's get_all_tensor mode); "
                         "by default the result of a conv that only feeds the add fused into it "
                         "is not written")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB read + 256 MiB write kernel (relu) so HBM "
                         "counters can be scaled against a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (--gpus %d refused); the path shards "
                 "by batch with no exchange step between GPUs" % args.gpus)

    import numpy as np
    from tpu_compiler_amd import graphs, module

    graph_fn = graphs.CONFIGS[args.config]
    g = graph_fn(batch=args.batch) if args.batch > 0 else graph_fn()
    batch = g.input_op().shape[0]
    if not args.tiles and not args.autotune and not args.save_tiles and args.batch <= 0:
        recorded = os.path.join(ROOT, RECORDED_TILES.get(args.config, ""))
        if os.path.isfile(recorded):
            args.tiles = recorded
    if args.tiles:
        from tpu_compiler_amd import capi
        tile_names = []
        while capi.bind().tpuhip_conv2d_tile_name(len(tile_names)):
            tile_names.append(capi.bind().tpuhip_conv2d_tile_name(len(tile_names)).decode())
        for name, algo in json.load(open(args.tiles)).items():
            if algo in tile_names:
                g.by_name[name].attrs["algo"] = 16 + tile_names.index(algo)
    m = module(device=0)
    m.set_option("keep_all_tensors", 1 if args.keep_all else 0)
    m.load(g)
    m.set_tensor(g.input_op().name, g.input_op().data.astype(np.float32))
    lib, ctxh = m.lib, m.context_handle()

    for _ in range(max(args.warmup, 1)):
        m.invoke()
    m.sync()
    if args.save_tiles:
        json.dump({name: algo for name, algo in m.kernels() if algo.startswith("mfma")},
                  open(args.save_tiles, "w"))

    if args.copy_calibration:
        from tpu_compiler_amd import capi
        cal = capi.Context(0)
        n = 256 << 20
        src, dst = cal.malloc(n), cal.malloc(n)
        cal._ck(cal.lib.tpuhip_memset(cal.h, src, 1, n))
        for _ in range(3):
            cal._ck(cal.lib.tpuhip_relu_i8(cal.h, src, dst, n))
        cal.sync()
        cal.free(src)
        cal.free(dst)
        cal.close()

    import ctypes as C
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.tpuhip_event_create(ctxh, C.byref(e0))
    lib.tpuhip_event_create(ctxh, C.byref(e1))
    m.sync()
    t0 = time.perf_counter()
    lib.tpuhip_event_record(ctxh, e0)
    for _ in range(args.steps):
        m.invoke()
    lib.tpuhip_event_record(ctxh, e1)
    m.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ev_ms = C.c_float()
    lib.tpuhip_event_elapsed_ms(ctxh, e0, e1, C.byref(ev_ms))
    ms_per_step = wall_ms / args.steps
    images_per_s = batch / (ms_per_step / 1e3)
    total_ops = 2.0 * g.macs
    tops = total_ops / (ms_per_step / 1e3) / 1e12

    # per-kernel times, HIP events on the stream the kernels run on
    rows = m.time_kernels(iters=max(5, min(args.steps, 20)))
    by_algo = {}
    algo_of = {name: algo for name, algo, _ in rows}
    ms_of = {name: ms for name, algo, ms in rows}
    # an eltwise add that launched nothing rides in the epilogue of the later of its conv inputs
    order = {op.name: i for i, op in enumerate(g.ops)}
    readers = {}
    for op in g.ops:
        for i in op.inputs:
            readers[i] = readers.get(i, 0) + 1
    fused_add = {}
    for op in g.ops:
        if op.type == "tpu.eltwise_add" and ms_of.get(op.name, 1) == 0:
            convs = [i for i in op.inputs if g.by_name[i].type == "tpu.conv_2d"]
            if convs:
                fused_add[max(convs, key=lambda n: order[n])] = op
    # likewise a max pool that launched nothing runs inside its producing conv's launch
    fused_pool = {op.inputs[0]: op for op in g.ops
                  if op.type == "tpu.pool_max_2d" and ms_of.get(op.name, 1) == 0
                  and g.by_name[op.inputs[0]].type == "tpu.conv_2d"}
    for name, algo, ms in rows:
        op = g.by_name[name]
        if op.type in ("tpu.conv_2d", "tpu.fully_connected"):
            # a conv that runs inside the launch of another ("with <name>") counts towards that launch
            rides = algo.startswith("with ")
            key = algo_of[algo[5:]] if rides else algo
            d = by_algo.setdefault(key, {"ms": 0.0, "ops": 0.0, "bytes": 0.0, "launches": 0})
            d["ms"] += ms
            d["ops"] += 2.0 * op.macs
            add = fused_add.get(name)
            pool = fused_pool.get(name)
            stored = (args.keep_all or (add is None and pool is None) or readers.get(name, 0) > 1
                      or name in g.outputs)
            d["bytes"] += conv_bytes(op, g, add, stored) - (int(np.prod(g.by_name[op.inputs[0]].shape)) if rides else 0)
            if pool is not None:
                d["bytes"] += int(np.prod(pool.shape))
            d["launches"] += 0 if rides else 1
    mfma = {k: v for k, v in by_algo.items() if k.startswith("mfma")}
    conv_ms = sum(v["ms"] for v in mfma.values())
    conv_ops = sum(v["ops"] for v in mfma.values())
    dom_name, dom = max(mfma.items(), key=lambda kv: kv[1]["ms"]) if mfma else (None, None)
    roofline = None
    if dom:
        achieved = dom["ops"] / (dom["ms"] / 1e3) / 1e12
        family = next((k for pre, k in (("mfma_chain_", "conv_chain_kernel"), ("mfma_pw_", "conv_pw_kernel"), ("mfma_patch2_", "conv_patch2_kernel"),
                                        ("mfma_patch_", "conv_patch_kernel"), ("mfma_reg_", "conv_mfma_reg_kernel"),
                                        ("mfma_splitk_", "conv_mfma_splitk_kernel")) if dom_name.startswith(pre)),
                      "conv_mfma_kernel")
        roofline = {"bound": "mfma", "kernel": "%s [tile %s]" % (family, dom_name),
                    "achieved": round(achieved, 2), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                    "frac": round(achieved / PEAK_INT8_TOPS, 4), "traffic": None,
                    "launches": dom["launches"],
                    "avg_launch_us": round(dom["ms"] * 1e3 / dom["launches"], 2),
                    "all_mfma_conv_layers": {
                        "achieved": round(conv_ops / (conv_ms / 1e3) / 1e12, 2),
                        "frac": round(conv_ops / (conv_ms / 1e3) / 1e12 / PEAK_INT8_TOPS, 4),
                        "ms": round(conv_ms, 4)}}
        # the same launches against the other roof: below the ridge (peak ops / peak bytes) a kernel that
        # moved only its algorithmic bytes at the HBM peak would still be slower than its MFMAs
        intensity = dom["ops"] / dom["bytes"]
        ridge = PEAK_INT8_TOPS * 1e12 / (PEAK_HBM_GBS * 1e9)
        gbs = dom["bytes"] / (dom["ms"] / 1e3) / 1e9
        roofline["against_hbm"] = {"ops_per_byte": round(intensity, 1), "ridge_ops_per_byte": round(ridge, 1),
                                   "lower_roof": "hbm" if intensity < ridge else "mfma",
                                   "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                   "frac": round(gbs / PEAK_HBM_GBS, 4)}
    # HBM bytes per launch of that kernel, from the committed rocprofv3 counter passes
    # (FETCH_SIZE + WRITE_SIZE, scaled against a plain copy kernel) of this same workload
    traffic_file = os.path.join(ROOT, "profiles", "resnet50_b32_bench_traffic.json")
    if roofline and args.config == "cfg3" and os.path.exists(traffic_file):
        t = json.load(open(traffic_file))["kernels"].get(dom_name)
        if t:
            roofline["traffic"] = int((t["fetch_KiB"] + t["write_KiB"]) * 1024)
            roofline["traffic_unit"] = "bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, profiles/)"
            roofline["algorithmic_bytes"] = int(dom["bytes"] / dom["launches"])
    # bandwidth-bound ops: algorithmic bytes (int8 inputs + output once) over their time
    hbm_bytes = hbm_ms = 0.0
    for name, algo, ms in rows:
        op = g.by_name[name]
        if op.type in ("tpu.conv_2d", "tpu.fully_connected", "tpu.input") or ms <= 0:
            continue
        hbm_bytes += sum(int(np.prod(g.by_name[i].shape)) for i in op.inputs) + int(np.prod(op.shape))
        hbm_ms += ms
    # what one op per launch can reach at best: every launch's algorithmic bytes at the HBM peak (or its
    # operations at the MFMA peak, whichever takes longer) behind one launch floor each
    floor_ms, n_launches, graph_bytes = 0.0, 0, 0.0
    for d in by_algo.values():
        floor_ms += max(d["bytes"] / (PEAK_HBM_GBS * 1e9), d["ops"] / (PEAK_INT8_TOPS * 1e12)) * 1e3
        n_launches += d["launches"]
        graph_bytes += d["bytes"]
    n_other = sum(1 for name, algo, ms in rows
                  if ms > 0 and g.by_name[name].type not in ("tpu.conv_2d", "tpu.fully_connected", "tpu.input"))
    floor_ms += hbm_bytes / (PEAK_HBM_GBS * 1e9) * 1e3
    n_launches += n_other
    graph_bytes += hbm_bytes
    launch_ms = n_launches * LAUNCH_FLOOR_US / 1e3
    graph_floor = {"launches": n_launches, "algorithmic_bytes": int(graph_bytes),
                   "data_ms": round(floor_ms, 4), "launch_ms": round(launch_ms, 4),
                   "floor_ms": round(floor_ms + launch_ms, 4),
                   "step_over_floor": round(ms_per_step / (floor_ms + launch_ms), 2),
                   "what": "per launch max(algorithmic bytes at %g GB/s, operations at %g TOP/s) + %.1f us "
                           "(an empty dependent launch)" % (PEAK_HBM_GBS, PEAK_INT8_TOPS, LAUNCH_FLOOR_US)}
    if args.per_layer:
        for name, algo, ms in rows:
            op = g.by_name[name]
            macs = getattr(op, "macs", 0)
            nbytes = sum(int(np.prod(g.by_name[i].shape)) for i in op.inputs) + int(np.prod(op.shape))
            print("%-22s %-18s %-18s %9.2f us %8.1f TOP/s %8.1f GB/s" %
                  (name, op.type, algo, ms * 1e3, 2 * macs / (ms / 1e3) / 1e12 if ms > 0 else 0,
                   nbytes / (ms / 1e3) / 1e9 if ms > 0 else 0),
                  file=sys.stderr)

    out = {
        "metric": "images_per_sec", "value": round(images_per_s, 1), "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "%s: %s INT8 graph, batch %d, %s input, random-init seeded weights"
                               % (args.config, g.name, batch,
                                  "x".join(str(v) for v in g.input_op().shape[1:])),
                   "global_batch": batch,
                   "tensors_written": "all" if args.keep_all else
                                      "all but the conv results consumed only by the add or max pool fused into their launch",
                   "conv_tiles": ("recorded: " + os.path.relpath(args.tiles, ROOT)) if args.tiles else
                                 "timed on first use"},
        "tops": round(tops, 2),
        "ops_per_step": total_ops,
        "event_ms_per_step": round(ev_ms.value / args.steps, 4),
        "roofline": roofline,
        "graph_floor": graph_floor,
        "hbm_bound_ops": None if hbm_ms <= 0 else {
            "achieved": round(hbm_bytes / (hbm_ms / 1e3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(hbm_bytes / (hbm_ms / 1e3) / 1e9 / PEAK_HBM_GBS, 4), "ms": round(hbm_ms, 4)},
    }
    if args.host_io:
        # the boundary as pymlir's run(x) uses it: fp32 NCHW in host memory -> device int8 and back
        x_host = g.input_op().data.astype(np.float32)
        in_name = g.input_op().name
        for _ in range(2):
            m.set_tensor(in_name, x_host)
            m.invoke()
            outs = [m.get_tensor(name) for name in g.outputs]
        m.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            m.set_tensor(in_name, x_host)
            m.invoke()
            outs = [m.get_tensor(name) for name in g.outputs]
        ms_io = (time.perf_counter() - t0) * 1e3 / args.steps
        out["host_io"] = {"ms_per_step": round(ms_io, 4), "images_per_s": round(batch / (ms_io / 1e3), 1),
                          "host_bytes_in": int(x_host.nbytes), "host_bytes_out": int(sum(o.nbytes for o in outs)),
                          "what": "set_tensor(fp32, caller's pageable buffer) + invoke + get_tensor(fp32) per step"}
        if g.input_op().data.dtype == np.int8:
            # the same with the int8 entry points at both ends, for callers that hold bytes already
            x8 = np.ascontiguousarray(g.input_op().data)
            for _ in range(2):
                m.set_tensor_i8(in_name, x8)
                m.invoke()
                outs = [m.get_tensor_i8(name) for name in g.outputs]
            m.sync()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                m.set_tensor_i8(in_name, x8)
                m.invoke()
                outs = [m.get_tensor_i8(name) for name in g.outputs]
            ms_i8 = (time.perf_counter() - t0) * 1e3 / args.steps
            out["host_io"]["int8"] = {"ms_per_step": round(ms_i8, 4),
                                      "images_per_s": round(batch / (ms_i8 / 1e3), 1),
                                      "host_bytes_in": int(x8.nbytes),
                                      "host_bytes_out": int(sum(o.nbytes for o in outs)),
                                      "what": "set_tensor_i8 + invoke + get_tensor_i8 per step"}
    # the reference's get_all_tensor mode beside the headline: every tensor of the graph written
    mk = None
    if not args.keep_all:
        mk = module(device=0)
        mk.set_option("keep_all_tensors", 1)
        mk.load(g)
        mk.set_tensor(g.input_op().name, g.input_op().data.astype(np.float32))
        for _ in range(max(args.warmup, 1)):
            mk.invoke()
        mk.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            mk.invoke()
        mk.sync()
        ms_keep = (time.perf_counter() - t0) * 1e3 / args.steps
        out["keep_all"] = {"ms_per_step": round(ms_keep, 4), "images_per_s": round(batch / (ms_keep / 1e3), 1),
                           "what": "every tensor of the graph written, as the reference's get_all_tensor mode needs"}
    out["parity_checked"] = False
    if not args.no_cpu_baseline:
        sample = min(batch, {"cfg1": 64, "cfg2": 16, "cfg3": 32, "cfg4": 64, "cfg5": 2}[args.config])
        want = {}
        out["cpu_baseline"] = cpu_baseline(graph_fn, sample, keep_results=want)
        # parity, outside the timed region: the outputs of the timed module, and every tensor of the
        # keep-all module, against the oracle on the first `sample` images (ops are independent across
        # the batch, and the generators give image i the same data whatever the batch)
        guards = want.pop("__guards__")
        full = graph_fn(batch=sample) if sample != batch else g
        same_input = np.array_equal(full.input_op().data, g.input_op().data[:sample])
        outputs_ok = same_input and all(
            np.array_equal(m.get_tensor_i8(name)[:sample], want[name]) for name in g.outputs)
        src = mk if mk is not None else m
        exact = sum(1 for op in g.ops
                    if np.array_equal(src.get_tensor_i8(op.name)[:sample], want[op.name].reshape((sample,) + tuple(op.shape[1:]))))
        out["parity_checked"] = bool(outputs_ok)
        out["parity"] = {"outputs_equal_oracle": bool(outputs_ok), "layers_exact": exact, "layers_total": len(g.ops),
                         "images_checked": sample,
                         "fp32_guard_held": bool(max(guards.values()) < (1 << 24)) if guards else None}
        try:
            out["parity"]["activations"] = activation_stats(g.ops, want, guards)
        except Exception as e:      # statistics only: never in the way of the line
            out["parity"]["activations"] = {"error": str(e)}
    if mk is not None:
        mk.close()
    m.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
