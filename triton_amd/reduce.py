"""Reduction over one axis with optional mask and scale (reduce.py:1135-1157 of
the reference); used as the top-k combine: y.view(T, k, N) -> sum over k."""
from typing import Optional

import torch

from . import _lib


def _bstrides(t: Optional[torch.Tensor], shape3):
    """Strides of `t` broadcast to [S0, R, S1] (size-1 axes get stride 0)."""
    if t is None:
        return (0, 0, 0)
    assert t.ndim == 3, "mask / scale must have the rank of x"
    out = []
    for d in range(3):
        assert t.shape[d] in (1, shape3[d]), f"cannot broadcast {tuple(t.shape)} to {tuple(shape3)}"
        out.append(0 if t.shape[d] == 1 else t.stride(d))
    return tuple(out)


def reduce(x: torch.Tensor, dim: int, mask: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
           x_mxscale=None, x_flex=None, x_global_scale=None, y: Optional[torch.Tensor] = None,
           y_dtype: Optional[torch.dtype] = None, y_flex=None, y_flex_saturate_inf: bool = False, y_has_mx=None,
           y_mx_scale_dtype=None, y_microblock_size: int = 32, y_value_pack_factor: int = 1, postprocess_fn1=None,
           postprocess_fn2=None, unpadded_batch_size=None):
    """Returns (y, None): y = sum over `dim` of where(mask, x*scale, 0), accumulated
    in float32 in index order and cast to y_dtype (default x.dtype)."""
    def _flex_used(f):
        return f is not None and any(getattr(f, n, None) is not None for n in ("scale", "expected_scale", "actual_scale"))
    if _flex_used(y_flex) or x_global_scale is not None or postprocess_fn1 is not None or postprocess_fn2 is not None \
            or unpadded_batch_size is not None:
        raise NotImplementedError("output flex / global scale / postprocess variants of reduce are not built")
    _lib.require_gpu(x, "x")
    dim = dim % x.ndim
    x_flex_scale = getattr(x_flex, "scale", None) if x_flex is not None else None
    if x_flex_scale is not None:
        # one float32 factor on the input: folded into the per-element scale operand
        fs = x_flex_scale.to(torch.float32).reshape((1, ) * x.ndim)
        scale = fs if scale is None else scale.to(torch.float32) * fs
    if x_mxscale is not None:
        # microscaled input and output (reduce.py:1185-1206 of the reference): dequantise along the last axis, sum in
        # float32, quantise the sum to MXFP8 along the last axis -- three launches of the kernels of this library
        from .numerics_details.mxfp import downcast_to_mxfp, upcast_from_mxfp
        assert dim != x.ndim - 1, "the microscaled axis cannot be reduced"
        assert y is None and y_has_mx in (None, True) and y_microblock_size == 32 and y_value_pack_factor == 1
        x32 = upcast_from_mxfp(x, x_mxscale, torch.float32, axis=-1)
        y32, _ = reduce(x32, dim, mask=mask, scale=scale, y_dtype=torch.float32)
        return downcast_to_mxfp(y32, torch.float8_e4m3fn, axis=-1)
    if y_has_mx:
        raise NotImplementedError("a microscaled output needs a microscaled input (as in the reference's torch twin)")
    if x.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        raise NotImplementedError("fp8 inputs without block scales are not built")
    lead = 1
    for s in x.shape[:dim]:
        lead *= s
    tail = 1
    for s in x.shape[dim + 1:]:
        tail *= s
    R = x.shape[dim]
    if not x.is_contiguous():
        x = x.contiguous()
    if mask is None and scale is None and y is None and R >= 512 and lead * tail <= (1 << 18):
        # a long axis over few outputs: a thread of the kernel walks the whole axis, so it is cut into chunks that
        # are summed side by side (float32 partial sums), then the chunks are summed
        chunks = next((c for c in (64, 32, 16, 8) if R % c == 0), 0)
        if chunks:
            part, _ = reduce(x.view(lead, chunks, R // chunks, tail), 2, y_dtype=torch.float32)
            out, _ = reduce(part, 1, y_dtype=y_dtype or x.dtype)
            return out.view([*x.shape[:dim], *x.shape[dim + 1:]]), None
    x3 = x.view(lead, R, tail)

    def to3(t):
        if t is None:
            return None
        assert t.ndim == x.ndim
        lead_t = 1
        for s in t.shape[:dim]:
            lead_t *= s
        tail_t = 1
        for s in t.shape[dim + 1:]:
            tail_t *= s
        if lead_t not in (1, lead) or tail_t not in (1, tail):
            t = t.expand(x.shape)
            lead_t, tail_t = lead, tail
        return t.reshape(lead_t, t.shape[dim], tail_t)

    mask3, scale3 = to3(mask), to3(scale)
    if mask3 is not None:
        mask3 = mask3.to(torch.bool).view(torch.uint8) if mask3.dtype != torch.uint8 else mask3
    if scale3 is not None and scale3.dtype != torch.float32:
        scale3 = scale3.to(torch.float32)
    y_dtype = y_dtype or x.dtype
    out_shape = [*x.shape[:dim], *x.shape[dim + 1:]]
    if y is None:
        y = torch.empty(out_shape, dtype=y_dtype, device=x.device)
    else:
        assert list(y.shape) == out_shape and y.is_contiguous() and y.dtype == y_dtype
    y2 = y.view(lead, tail)
    ms, ss = _bstrides(mask3, x3.shape), _bstrides(scale3, x3.shape)
    rc = _lib.lib().tamd_reduce(_lib.ptr(x3), _lib.dtype_code(x.dtype), lead, R, tail, x3.stride(0), x3.stride(1),
                                x3.stride(2), _lib.ptr(mask3), *ms, _lib.ptr(scale3), *ss, _lib.ptr(y2),
                                _lib.dtype_code(y_dtype), y2.stride(0), y2.stride(1), _lib.stream_ptr(x.device))
    _lib.check(rc, "reduce")
    return y, None
