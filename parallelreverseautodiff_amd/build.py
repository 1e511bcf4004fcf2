"""Builds libprad_hip.so for gfx950 with hipcc, in-tree.

Usage: ``python -m parallelreverseautodiff_amd.build`` (or ``build_library()`` from Python).
The shared library is the whole product: a C ABI (include/prad_hip.h) over hand-written HIP
kernels.  Nothing here depends on PyTorch.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libprad_hip.so")
SOURCES = ["gemm.hip", "gemm_skinny.hip", "gemm_tall.hip", "elementwise.hip", "optim.hip", "matmul_sum.hip", "loss.hip", "head.hip", "lstm.hip", "lstm_seq.hip", "attention.hip", "norm.hip", "prad_hip.hip"]

# -packed-fp32-ops is switched off: the compiler must not form packed FP32 instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def build_library(verbose=False):
    """Compiles every HIP source and links libprad_hip.so next to this file."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        out = _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs)
    build_host_walk()
    return LIB_PATH


def build_host_walk():
    """libprad_hostwalk.so: a compiled caller of the C ABI (csrc/host_walk.cpp, host code only), used by the
    benchmark and one test to drive a training step operation by operation without an interpreter in between."""
    out = os.path.join(HERE, "libprad_hostwalk.so")
    _run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden", os.path.join(CSRC, "host_walk.cpp"), "-o", out,
          "-L" + HERE, "-lprad_hip", "-Wl,-rpath,$ORIGIN"])
    return out


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
