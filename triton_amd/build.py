"""Builds libtriton_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python -m triton_amd.build [--force]
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtriton_amd.so")
SOURCES = ["api.cpp", "mxfp.hip", "routing.hip", "elementwise.hip", "moe_matmul.hip", "moe_matmul_bf16.hip", "moe_matmul_f16.hip",
           "moe_matmul_fp8.hip", "moe_matmul_bf16_swiglu.hip", "moe_matmul_f16_swiglu.hip", "moe_matmul_fp8_swiglu.hip",
           "moe_matmul_fp8e5m2.hip", "moe_matmul_fp8e5m2_swiglu.hip", "moe_matmul_stream_fp8e5m2.hip",
           "moe_matmul_stream_bf16.hip", "moe_matmul_stream_f16.hip", "moe_matmul_stream_fp8.hip",
           "moe_matmul_w16_bf16.hip", "moe_matmul_w16_f16.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 math is switched off on purpose (device code only); the unroll limit is raised because the tile
# epilogues index their accumulators with loops that must unroll completely (up to 80 element rows per lane):
# at the default limit the largest ones stay rolled and the accumulators drop into scratch memory
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-mllvm", "-pragma-unroll-threshold=65536", "-Wno-unused-command-line-argument"]


EXTRA = os.environ.get("TAMD_EXTRA_HIPCC_FLAGS", "").split()  # e.g. -DTAMD_STREAM_WGS_PER_CU=1 for experiments


def _scratch_users(remarks):
    """Kernels that use scratch memory (register spills or arrays the compiler could not keep in registers),
    from the kernel-resource-usage remarks: [(mangled name, bytes per lane)]."""
    out, name = [], None
    for line in remarks.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and int(m.group(1)) > 0:
            out.append((name, int(m.group(1))))
    return out


def _scratch_instructions(src, names):
    """Number of scratch loads / stores in the generated code of the kernels `names` of one source (the device
    assembly is produced for this check only)."""
    asm = os.path.join(HERE, "build", os.path.splitext(src)[0] + ".check.s")
    cmd = [HIPCC, *FLAGS, *EXTRA, "-x", "hip", "--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", asm]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        return {}
    counts, cur = {}, None
    with open(asm) as f:
        for line in f:
            if line and not line[0].isspace() and line.rstrip().split(":")[0] in names and ":" in line:
                cur = line.split(":")[0]
                counts.setdefault(cur, 0)
            elif ".end_amdhsa_kernel" in line:
                cur = None
            elif cur is not None and re.search(r"\bscratch_(load|store)", line):
                counts[cur] += 1
    os.remove(asm)
    return counts


def _compile(src, obj):
    cmd = [HIPCC, *FLAGS, *EXTRA, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    if src.endswith(".hip"):
        cmd.append("-Rpass-analysis=kernel-resource-usage")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    # every kernel here is written to live in registers; one that falls into scratch memory still computes
    # the right values, several times slower, so the build is where it has to be caught
    spilled = _scratch_users(res.stderr)
    if spilled and not os.environ.get("TAMD_ALLOW_SCRATCH"):
        # a kernel may be given a small private segment without a single access to it (stack slots the register
        # allocator reserved and then did not need): what counts is whether its code touches scratch memory
        touching = _scratch_instructions(src, [n for n, _ in spilled])
        spilled = [(n, b) for n, b in spilled if touching.get(n, 1) > 0]
    if spilled and not os.environ.get("TAMD_ALLOW_SCRATCH"):
        os.remove(obj)
        raise RuntimeError(f"{src}: kernels using scratch memory: " + ", ".join(f"{n} ({b} B/lane)" for n, b in spilled))


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
