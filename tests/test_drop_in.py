"""`install_as_triton_kernels()`: every module path, callable, parameter name and dataclass field of the reference's
package that the hot path's callers use resolves to this package.  The expected names are data transcribed from the
reference's sources (tests/golden/reference_api.json, file:line beside every entry)."""
import dataclasses
import importlib
import inspect
import json
import os
import sys

import pytest

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_api.json")))


@pytest.fixture(scope="module")
def installed():
    import triton_amd
    before = {k: v for k, v in sys.modules.items() if k == "triton_kernels" or k.startswith("triton_kernels.")}
    triton_amd.install_as_triton_kernels()
    yield
    for k in [k for k in sys.modules if k == "triton_kernels" or k.startswith("triton_kernels.")]:
        if k not in before:
            del sys.modules[k]


def resolve(path):
    mod, name = path.rsplit(".", 1)
    return getattr(importlib.import_module(mod), name)


@pytest.mark.parametrize("path", sorted(GOLDEN["callables"]))
def test_callable_keeps_the_reference_parameters(installed, path):
    fn = resolve(path)
    want = GOLDEN["callables"][path]["params"]
    got = [p.name for p in inspect.signature(fn).parameters.values()
           if p.kind not in (inspect.Parameter.VAR_KEYWORD, inspect.Parameter.VAR_POSITIONAL)]
    # same names in the same order; a trailing **kwargs (convert_layout) and extra keyword-only options are allowed
    assert got[:len(want)] == want, f"{path} ({GOLDEN['callables'][path]['at']}): {got} vs {want}"


@pytest.mark.parametrize("module", sorted(GOLDEN["names"]))
def test_module_exports_the_reference_names(installed, module):
    mod = importlib.import_module(module)
    assert mod.__name__.startswith("triton_amd"), "the module is this package's"
    missing = [n for n in GOLDEN["names"][module]["names"] if not hasattr(mod, n)]
    assert not missing, f"{module} ({GOLDEN['names'][module]['at']}) lacks {missing}"


@pytest.mark.parametrize("path", sorted(GOLDEN["dataclass_fields"]))
def test_dataclass_fields_match_field_for_field(installed, path):
    cls = resolve(path)
    assert [f.name for f in dataclasses.fields(cls)] == GOLDEN["dataclass_fields"][path]["fields"]


def test_from_imports_as_the_reference_harness_writes_them(installed):
    """The import lines of bench/bench_mlp.py:8-21 of the reference that concern one GPU."""
    from triton_kernels.matmul import FlexCtx, FnSpecs, FusedActivation, PrecisionConfig, matmul  # noqa: F401
    from triton_kernels.matmul_details.opt_flags import scoped_opt_flags_constraints  # noqa: F401
    from triton_kernels.numerics import InFlexData  # noqa: F401
    from triton_kernels.numerics_details.mxfp import MXFP_BLOCK_SIZE, downcast_to_mxfp  # noqa: F401
    from triton_kernels.reduce import reduce  # noqa: F401
    from triton_kernels.swiglu import swiglu_fn  # noqa: F401
    from triton_kernels.target_info import get_cdna_version
    from triton_kernels.tensor import FP4, convert_layout, make_ragged_tensor_metadata, wrap_torch_tensor  # noqa: F401
    from triton_kernels.tensor_details import layout
    from triton_kernels.topk import topk  # noqa: F401
    assert layout.make_default_matmul_mxfp4_w_scale_layout(mx_axis=1).name == "CDNA4_SCALE"
    assert get_cdna_version() in (-1, 3, 4)  # -1 without a GPU
