"""Builds libhemm.so (HIP kernels + C ABI + C++ host layer) for gfx950 with hipcc, in-tree."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhemm.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wno-unused-value",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "host", "*.cpp")))


def _compile(src):
    obj = os.path.splitext(src)[0] + ".o"
    inc = ["-I", os.path.join(HERE, "..", "include"), "-I", CSRC, "-I", os.path.join(CSRC, "host")]
    cmd = [HIPCC] + FLAGS + inc + ["-c", src, "-o", obj]
    if src.endswith(".cpp"):
        # host layer: no fused multiply-adds, so the embedding FFT rounds the same everywhere
        cmd = [HIPCC] + FLAGS + ["-x", "hip", "-ffp-contract=off"] + inc + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj


def build(verbose=False):
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-o", LIB] + objs,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    build_examples(verbose)
    return LIB


def build_examples(verbose=False):
    """C++ callers of the host layer, compiled as plain C++ (no HIP) and linked with libhemm.so only."""
    ex = os.path.join(HERE, "examples")
    for src in sorted(glob.glob(os.path.join(ex, "*.cpp"))):
        out = os.path.splitext(src)[0]
        cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", src, "-I", os.path.join(CSRC, "host"),
               "-I", os.path.join(HERE, "..", "include"), "-L", HERE, "-lhemm", "-L/opt/rocm/lib",
               "-Wl,-rpath-link,/opt/rocm/lib", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath,/opt/rocm/lib", "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("example build failed for %s:\n%s" % (src, r.stderr))
        if verbose:
            print("built", out)


if __name__ == "__main__":
    build(verbose=True)
