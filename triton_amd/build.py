"""Builds libtriton_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python -m triton_amd.build [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtriton_amd.so")
SOURCES = ["api.cpp", "mxfp.hip", "routing.hip", "elementwise.hip", "moe_matmul.hip", "moe_matmul_bf16.hip", "moe_matmul_f16.hip",
           "moe_matmul_fp8.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 math is switched off on purpose (device code only)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


EXTRA = os.environ.get("TAMD_EXTRA_HIPCC_FLAGS", "").split()  # e.g. -DTAMD_STREAM_WGS_PER_CU=1 for experiments


def _compile(src, obj):
    cmd = [HIPCC, *FLAGS, *EXTRA, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")


def build(force=True, verbose=False):
    """Compiles every source and links the shared library. Returns its path."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(objdir, os.path.splitext(s)[0] + ".o") for s in srcs]
    deps = [os.path.join(CSRC, "common.h"), os.path.join(CSRC, "moe_matmul_impl.h"), os.path.join(CSRC, "moe_matmul_stream.h"), os.path.join(CSRC, "moe_matmul_dense.h"),
            os.path.join(HERE, "..", "include", "triton_amd.h")]
    todo = []
    for s, o in zip(srcs, objs):
        newest = max(os.path.getmtime(p) for p in [os.path.join(CSRC, s), *deps])
        if force or not os.path.exists(o) or os.path.getmtime(o) < newest:
            todo.append((s, o))
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(todo)))) as ex:
        list(ex.map(lambda so: _compile(*so), todo))
    if todo or not os.path.exists(LIB):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB} ({len(todo)} objects recompiled)")
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
