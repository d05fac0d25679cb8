"""Interleaved SwiGLU (swiglu.py of the reference): gate = even columns, linear =
odd columns, out = gate*sigmoid(alpha*gate) * (linear + 1) with clamping."""
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from .numerics import InFlexData, OutFlexData


@dataclass(frozen=True)
class FlexCtx:
    out_data: OutFlexData = OutFlexData()
    inp_data: InFlexData = InFlexData()
    saturate_inf: bool = False


@dataclass(frozen=True)
class PrecisionConfig:
    limit: Optional[float]
    flex_ctx: FlexCtx = FlexCtx()


def swiglu_fn(*_args, **_kwargs):
    """Placeholder carried in FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2);
    the fused epilogue is selected by the spec's name."""
    raise RuntimeError("swiglu_fn is a tag for the fused matmul epilogue, not a callable")


def swiglu(a: torch.Tensor, alpha: float, precision_config: PrecisionConfig, routing_data=None):
    _lib.require_gpu(a, "a")
    fc = precision_config.flex_ctx
    if fc.inp_data.scale is not None or fc.out_data.expected_scale is not None or fc.out_data.actual_scale is not None:
        raise NotImplementedError("flexpoint scaling in the standalone swiglu is not built")
    assert a.stride(-1) == 1
    assert a.shape[-1] % 2 == 0
    N = a.shape[-1]
    a2 = a.reshape(-1, N)
    M = a2.shape[0]
    out = torch.empty((M, N // 2), dtype=a.dtype, device=a.device)
    limit = precision_config.limit
    rc = _lib.lib().tamd_swiglu(_lib.ptr(a2), _lib.dtype_code(a.dtype), M, N // 2, a2.stride(0), _lib.ptr(out),
                                out.stride(0), float(alpha), float(limit if limit is not None else 0.0),
                                int(limit is not None), _lib.stream_ptr(a.device))
    _lib.check(rc, "swiglu")
    return out.view(*a.shape[:-1], N // 2)
