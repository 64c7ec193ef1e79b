#!/usr/bin/env python3
"""Writes tests/golden/opgraphs/: the reference's fp32 op-test graphs
(lib/Dialect/TPU/Backend/test/*.mlir) after THIS repository's calibration-import + quantisation
pass, as the quantized .mlir text this repository's printer emits plus the quantized weight file.

The reference fills such graphs with unseeded random weights when it runs them
(lib/Dialect/TPU/Analysis/GenFakeWeightNpz.cpp:56-57), so nothing of its runs can be a vector;
the stand-in is a seeded generator: normal(0, 0.2) weights of the shapes the graph declares and
one uniform(0.8, 4.0) threshold per op as the calibration table.  Needs /root/reference (this
container only); the GPU tests read only what is written here.

Weights are stored with their integer types (int8 filters, int32 biases, uint32 rshift /
multiplier), compressed: the library's reader widens them to the float-stored form.

  python tests/golden/make_opgraph_fixtures.py
"""
import os
import pathlib
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from tpu_compiler_amd import capi, quantize as Q  # noqa: E402

REF_TESTS = "/root/reference/lib/Dialect/TPU/Backend/test"
OUT = os.path.join(HERE, "opgraphs")
# the op-test graphs whose every op this build's INT8 path covers.  Left out: pixel_shuffle for its
# 23 MB of weights; crop, whose second op asks for channels 32..41 of a 16-channel tensor (the
# reference only compiles that graph; an interpreter would read past the input, this library refuses)
GRAPHS = ["conv", "conv_1_oc", "deconv", "fc", "eltwise_add", "avg_pool", "max_pool", "relu", "concat",
          "broadcast_mul", "permute", "reorg", "reverse", "tile",
          "broadcast", "conv_large_w", "swap_channel", "permute_large", "lrn", "fc_large"]
# A quantized tensor of more than this many bytes is not stored: the weight file holds a descriptor
# "<name>__seeded" = [seed, 100 * sigma, shape...] instead, and materialize() draws the tensor --
# rint(normal(0, sigma)) clipped to +-127, the statistics of the quantized tensor it stands for --
# for the HIP path and the oracle alike (fc_large: a 23501 x 512 filter, 12 MB).
SEEDED_ABOVE = 1 << 20
_STORAGE = {"INT8": np.int8, "UINT8": np.uint8, "INT16": np.int16, "INT32": np.int32, "UINT32": np.uint32}


def prepare(name, tmp, rng):
    """the fp32 graph as the reference holds it, seeded weights under the file name it asks for,
    a calibration table with one seeded threshold per op"""
    path = tmp / (name + ".mlir")
    text = open(os.path.join(REF_TESTS, name + ".mlir")).read()
    lrn_thr = np.random.default_rng(77).uniform(0.8, 4.0)   # (a stream of its own: the other graphs' draws stay as they were)
    if name == "lrn":
        # the reference splits an LRN into three ops for calibration and folds their thresholds back
        # into the op as threshold_parts (Quantization.cpp:296-313); the test graph holds the unsplit
        # op, so the three are stated here from the op's own constants and its input's threshold T:
        # max of alpha / size * x^2, of its window sum, and of (k + sum)^-beta
        alpha, size = 9.99999974e-5, 5
        parts = (alpha / size * lrn_thr ** 2, alpha * lrn_thr ** 2, 1.0)
        text = text.replace("sum_rshift = 0 : i32}", "sum_rshift = 0 : i32, threshold_parts = [%.9g : f32, %.9g : f32, %.9g : f32]}" % parts)
        assert "threshold_parts" in text
    path.write_text(text)
    weights, wfile, ops = {}, None, []
    for line in capi.mlir_describe(str(path)).splitlines():
        w = line.split(" ")
        if w[0] == "weight_file":
            wfile = w[1]
        elif w[0] == "weight":
            weights[w[1]] = rng.normal(0, 0.2, [int(v) for v in w[3][1:-1].split(",") if v]).astype(np.float32)
        elif w[0] == "op":
            ops.append(w[2])
    if weights:
        np.savez(tmp / wfile, **weights)
    table = tmp / (name + "_table")
    table.write_text("".join("%s %.5f\n" % (op, lrn_thr if (name == "lrn" and op == "relu") else rng.uniform(0.8, 4.0))
                             for op in ops))
    return path, table


def write_one(name, tmp):
    rng = np.random.default_rng(1000 + sum(map(ord, name)))
    path, table = prepare(name, tmp, rng)
    out = tmp / (name + "_int8.mlir")
    problems = Q.quantize_files(path, table, out)
    assert problems == [], (name, problems)
    text = out.read_text()
    storage = {}
    for line in capi.mlir_describe(str(out)).splitlines():
        w = line.split(" ")
        if w[0] == "weight":
            storage[w[1]] = w[2]
    open(os.path.join(OUT, name + "_int8.mlir"), "w").write(text)
    wpath = tmp / (name + "_int8_weights.npz")
    wbytes = 0
    if wpath.exists():
        typed = {}
        with np.load(wpath) as z:
            for k in z.files:
                t = _STORAGE.get(storage.get(k, "NONE"))
                a = z[k]
                a = a.astype(t) if t is not None and np.array_equal(a.astype(t).astype(np.float32), a) else a
                if a.nbytes > SEEDED_ABOVE:
                    assert a.dtype == np.int8, (k, a.dtype)
                    sigma = float(np.std(a.astype(np.float32)))
                    typed[k + "__seeded"] = np.array([1000 + sum(map(ord, k)), round(100 * sigma)] + list(a.shape), np.int64)
                else:
                    typed[k] = a
        np.savez_compressed(os.path.join(OUT, name + "_int8_weights.npz"), **typed)
        wbytes = os.path.getsize(os.path.join(OUT, name + "_int8_weights.npz"))
    print(name, len(text), "bytes of text,", wbytes, "bytes of weights")


def materialize(name, dst_dir):
    """path of the stored quantized graph `name` with a complete weight file beside it: the stored
    files themselves, or -- where a tensor is held as a seeded descriptor -- copies under dst_dir
    with that tensor drawn"""
    src = os.path.join(OUT, name + "_int8.mlir")
    wsrc = os.path.join(OUT, name + "_int8_weights.npz")
    if not os.path.exists(wsrc):
        return src
    with np.load(wsrc) as z:
        if not any(k.endswith("__seeded") for k in z.files):
            return src
        full = {}
        for k in z.files:
            if k.endswith("__seeded"):
                seed, sigma100, *shape = [int(v) for v in z[k]]
                rng = np.random.default_rng(seed)
                full[k[:-len("__seeded")]] = np.clip(np.rint(rng.normal(0, sigma100 / 100.0, shape)), -127, 127).astype(np.int8)
            else:
                full[k] = z[k]
    os.makedirs(dst_dir, exist_ok=True)
    dst = os.path.join(str(dst_dir), name + "_int8.mlir")
    open(dst, "w").write(open(src).read())
    np.savez(os.path.join(str(dst_dir), name + "_int8_weights.npz"), **full)
    return dst


def main():
    os.makedirs(OUT, exist_ok=True)
    for name in GRAPHS:
        with tempfile.TemporaryDirectory(prefix="opgraph_") as tmpdir:
            write_one(name, pathlib.Path(tmpdir))


if __name__ == "__main__":
    main()
