"""Builds libes_km.so (the C-ABI kernel manager) for gfx950 with hipcc, in-tree.

    python -m einsummable_amd.build

hipcc cross-compiles without a GPU.  Every HIP translation unit is compiled with
packed-FP32 instruction selection disabled.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libes_km.so")
OBJ = os.path.join(HERE, "build")

SOURCES = [
    "ir.cc",
    "kernel_manager.cc",
    "c_api.cc",
    "exec_graph.cc", "memgraph_wire.cc", "pools.cc",
    "codegen.cc",
    "touch.hip",
    "static_workspace.hip",
    "transpose.hip",
    "contraction.hip",
    "complex_contraction.hip",
    "gemm_f16.hip",
    "gemm_f32.hip",
    "gemm_f64.hip",
]

COMMON = ["-std=c++17", "-O3", "-fPIC", "-Wall", "-Wno-unused-function"]
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    obj = os.path.join(OBJ, src + ".o")
    cmd = ["hipcc"] + COMMON + DEVICE + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    cmd = ["hipcc", "-shared", "-fPIC", "-Wl,-soname,libes_km.so", "-o", LIB] + objs + ["-lhiprtc"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
