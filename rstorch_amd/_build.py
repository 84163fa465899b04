"""Builds ``librstorch_hip.so`` (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

``python -m rstorch_amd._build`` or ``rstorch_amd._build.build_library()``.  The build is a
cross-compile: it needs no GPU.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(LIB_DIR, "librstorch_hip.so")

SOURCES = ["engine.hip", "gemm_f64.hip", "streaming.hip", "softmax_ce.hip", "rng_fill.hip",
           "ops.hip", "model.hip", "staging.hip", "static_scratch.hip"]

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # a*b+c stays two roundings, as in the reference's element-wise ndarray expressions
    "-ffp-contract=off",
    # packed FP32 instructions are not to be generated on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the backend is built with ROCm's hipcc for gfx950")
    return exe


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc()] + HIP_FLAGS + ["-c", os.path.join(CSRC_DIR, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build_library(verbose=False):
    """Compiles every source for gfx950 and links the shared library.  Always rebuilds."""
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES))
    for _, out in results:
        if out and verbose:
            print(out)
    objs = [o for o, _ in results]
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH] + objs
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
