"""Ahead-of-time build of libtango_hip.so for gfx950 (cross-compiles without a GPU).

The reference JIT-compiles its extension at import (cuda/kernels.py:12-16);
here the library is built once, in-tree, and only loaded at import.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtango_hip.so")
SOURCES = ["quantize.hip", "spmm.hip", "spmm_dense.hip", "sddmm.hip", "edge_softmax.hip", "qgemm.hip", "loss.hip", "attention.hip", "batchnorm.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # IEEE fp32 semantics: no contraction into FMA, default (correctly rounded) divide
    "-ffp-contract=off",
    # hipcc must not form packed-fp32 instructions on its own
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False):
    """Compile every HIP source and link the shared library.  Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = [os.path.join(LIB_DIR, s.replace(".hip", ".o")) for s in SOURCES]

    def one(pair):
        src, obj = pair
        return _run([HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        logs = list(ex.map(one, zip(SOURCES, objs)))
    logs.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs))
    if verbose:
        sys.stderr.write("\n".join(l for l in logs if l) + "\n")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
