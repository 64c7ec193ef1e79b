"""Builds libtpuhip.so (HIP kernels + C ABI + C++ host layer) for gfx950 with hipcc.

Run as ``python -m tpu_compiler_amd.build``.  hipcc cross-compiles, so no GPU is
needed to build.
"""
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libtpuhip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    srcs += sorted(glob.glob(os.path.join(CSRC, "host", "*.cpp")))
    return srcs


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS
    for s in sources():
        # .cpp host files are compiled as HIP too so they can include the runtime headers
        cmd += ["-x", "hip", s]
    cmd += ["-lz", "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "warning generated" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
