"""The C ABI library loads without a GPU and exports exactly what include/triton_amd.h declares; the ctypes
mirror of tamd_matmul_args has the header's field order.  No kernel is launched here."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "triton_amd.h")


def _header_text():
    text = open(HEADER).read()
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def _declared_functions():
    return sorted(set(re.findall(r"\b(tamd_\w+)\s*\(", _header_text())))


@pytest.fixture(scope="module")
def lib():
    from triton_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from triton_amd import build
        build.build()
    return _lib.lib()


def test_header_declares_the_path():
    names = _declared_functions()
    for need in ("tamd_topk_forward", "tamd_bitmatrix_metadata", "tamd_ragged_metadata", "tamd_routing_metadata",
                 "tamd_downcast_mxfp", "tamd_upcast_mxfp", "tamd_matmul", "tamd_reduce", "tamd_swiglu", "tamd_version"):
        assert need in names


def test_library_exports_every_declared_symbol(lib):
    from triton_amd import _lib
    declared = _declared_functions()
    assert sorted(_lib.EXPORTS) == declared
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.tamd_version() >= 1
    assert lib.tamd_error_string(-2).decode() != ""
    assert lib.tamd_error_string(-1).decode() != lib.tamd_error_string(-3).decode()


def test_matmul_args_mirror_matches_header():
    from triton_amd import _lib
    body = re.search(r"typedef struct\s*\w*\s*\{(.*?)\}\s*tamd_matmul_args\s*;", _header_text(), flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        m = re.match(r"(const\s+)?(\w+)\s*(\*?)\s*(.*)", decl)
        ctype = m.group(2)
        for part in m.group(4).split(","):
            part = part.strip()
            is_ptr = bool(m.group(3)) or part.startswith("*")
            fields.append((part.lstrip("* "), "ptr" if is_ptr else ctype))
    kinds = {C.c_void_p: "ptr", C.c_int: "int", C.c_int64: "int64_t", C.c_float: "float"}
    mirror = [(n, kinds[t]) for n, t in _lib.MatmulArgs._fields_]
    assert mirror == fields


def test_compiled_struct_size_matches_ctypes(tmp_path):
    from triton_amd import _lib
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include "triton_amd.h"\n'
                   'int main(void){printf("%zu %zu\\n", sizeof(tamd_matmul_args), '
                   '__builtin_offsetof(tamd_matmul_args, x_rows));return 0;}\n')
    exe = tmp_path / "sz"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    size, off = map(int, subprocess.check_output([str(exe)]).split())
    assert size == C.sizeof(_lib.MatmulArgs)
    assert off == _lib.MatmulArgs.x_rows.offset


def test_header_is_plain_c(tmp_path):
    src = tmp_path / "c.c"
    src.write_text('#include "triton_amd.h"\nint main(void){return 0;}\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                           str(src)])


def test_host_only_entry_points(lib):
    # pure host arithmetic: needs no device
    assert lib.tamd_bitmatrix_metadata_workspace(16384, 128) > 0
    assert lib.tamd_bitmatrix_metadata_workspace(0, 128) >= 0


def test_matmul_rejects_degenerate_problems_before_any_launch(lib):
    """Argument checks that return before the first HIP call (so they run without a device): a null argument block,
    negative sizes, and K == 0 with non-null pointers, which the kernels' K loops are not built for."""
    from triton_amd import _lib
    assert lib.tamd_matmul(None, None) == _lib.E_INVALID
    a = _lib.MatmulArgs()
    a.x, a.w, a.y, a.w_mx_scale = 0x1000, 0x2000, 0x3000, 0x4000  # never dereferenced on these paths
    a.x_dtype, a.w_dtype, a.y_dtype = _lib.BF16, _lib.MXFP4, _lib.BF16
    a.M, a.N, a.K, a.n_experts = 16, 256, 0, 1
    a.x_stride_m, a.w_stride_k, a.w_stride_n, a.w_mx_stride_k, a.w_mx_stride_n, a.y_stride_m = 0, 1, 0, 1, 0, 256
    assert lib.tamd_matmul(C.byref(a), None) == _lib.E_UNSUPPORTED
    a.K = -32
    assert lib.tamd_matmul(C.byref(a), None) == _lib.E_INVALID
    a.K, a.n_experts = 64, 0
    assert lib.tamd_matmul(C.byref(a), None) == _lib.E_INVALID
    a.n_experts, a.K = 1, 48  # not a whole number of 32-element scale groups
    assert lib.tamd_matmul(C.byref(a), None) == _lib.E_INVALID


def test_no_cpu_fallback_in_product():
    """The package never imports the oracle and refuses CPU tensors."""
    import torch
    import triton_amd
    from triton_amd.numerics_details.mxfp import downcast_to_mxfp
    assert not any(m == "oracle" or m.startswith("oracle.") for m in sys.modules
                   if "triton_amd" in (getattr(sys.modules[m], "__file__", "") or ""))
    pkg = os.path.dirname(triton_amd.__file__)
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f
    with pytest.raises(RuntimeError):
        downcast_to_mxfp(torch.zeros(1, 32), torch.uint8, axis=1)
