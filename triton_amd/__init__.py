"""MI355X-native quantized-MoE kernels behind the `triton_kernels` Python API.

Module layout follows the reference package so call sites keep their imports:
topk, tensor, routing, numerics, numerics_details.mxfp, matmul, swiglu, reduce,
matmul_details.opt_flags, target_info, tensor_details.layout (+ layout_details).  `install_as_triton_kernels()` registers this package
under the name `triton_kernels`.
"""
import sys

__version__ = "0.1.0"


def install_as_triton_kernels():
    """Makes `import triton_kernels[...]` resolve to this package."""
    import importlib
    me = sys.modules[__name__]
    sys.modules.setdefault("triton_kernels", me)
    for sub in ("tensor", "topk", "routing", "numerics", "numerics_details", "numerics_details.mxfp", "matmul",
                "matmul_details", "matmul_details.opt_flags", "swiglu", "reduce", "specialize", "testing",
                "tensor_details", "tensor_details.layout", "tensor_details.ragged_tensor",
                "tensor_details.bitmatrix", "tensor_details.dtype", "tensor_details.layout_details",
                "tensor_details.layout_details.base", "tensor_details.layout_details.strided",
                "tensor_details.layout_details.cdna4_scale", "target_info"):
        mod = importlib.import_module(f"{__name__}.{sub}")
        sys.modules.setdefault(f"triton_kernels.{sub}", mod)
    return me
