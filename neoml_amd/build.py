"""Builds libneoml_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc.

Usage: python -m neoml_amd.build
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libneoml_hip.so")

SOURCES = ["runtime.hip", "mem_pool.cpp", "vector_ops.hip", "blas_ops.hip", "dnn_ops.hip", "wide_ops.hip", "rare_ops.hip", "gemm_mfma.hip"]

# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU instructions
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fgpu-flush-denormals-to-zero",  # the reference CPU engine runs with FTZ + DAZ
    "-Wall", "-Wno-unused-function", "-Wno-pass-failed",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src):
    obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build_library(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES))
    objs = [r[0] for r in results]
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
