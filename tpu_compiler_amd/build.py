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


def _compile(args):
    hipcc, src, obj = args
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    # .cpp host files are compiled as HIP too so they can include the runtime headers
    cmd = [hipcc] + flags + ["-x", "hip", "-c", src, "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, res.returncode, res.stdout


def build(verbose=True, jobs=None):
    """Compiles every source to an object of its own (in parallel: one file holds most of the
    kernels and takes most of the time) and links them; objects go to a temporary directory."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = sources()
    jobs = jobs or max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", os.cpu_count() or 1)), 16))
    with tempfile.TemporaryDirectory(prefix="tpuhip_build_") as tmp:
        work = [(hipcc, s, os.path.join(tmp, "%02d_%s.o" % (i, os.path.basename(s)))) for i, s in enumerate(srcs)]
        if verbose:
            print("%s %s -c <%d sources>  (%d at a time)" % (hipcc, " ".join(HIPCC_FLAGS), len(srcs), jobs),
                  flush=True)
        with ThreadPoolExecutor(jobs) as pool:
            results = list(pool.map(_compile, work))
        log = []
        for src, rc, out in results:
            text = "\n".join(l for l in out.splitlines()
                             if "packed-fp32-ops" not in l and "warning generated" not in l)
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, text))
            if text.strip():
                log.append(text)
        link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + [w[2] for w in work] + ["-lz", "-o", LIB]
        res = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n" + res.stdout)
    if verbose and log:
        print("\n".join(log))
    return LIB


MICROBENCH = os.path.join(PKG, "machine_ceilings.bin")


def build_microbench(verbose=True):
    """The stand-alone program that measures the machine's ceilings (launch floor, copy bandwidth,
    MFMA peak, LDS and L2 bandwidth, vector-ALU issue rates): csrc/microbench/machine_ceilings.hip.
    Not linked into the library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    src = os.path.join(CSRC, "microbench", "machine_ceilings.hip")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", src, "-o", MICROBENCH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, res.stdout))
    return MICROBENCH


if __name__ == "__main__":
    if "--microbench" in sys.argv[1:]:
        print("built", build_microbench())
        sys.exit(0)
    build()
    print("built", LIB)
    sys.exit(0)
