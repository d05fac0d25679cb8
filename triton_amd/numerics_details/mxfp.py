"""downcast_to_mxfp / upcast_from_mxfp (numerics_details/mxfp.py of the reference)
over the gfx950 kernels."""
from enum import Enum

import torch

from .. import _lib
from ..tensor import FP4, Tensor, empty, torch_dtype_to_dtype, wrap_torch_tensor
from ..tensor_details.dtype import UINT8
from ..tensor_details.layout import StridedLayout

MXFP_BLOCK_SIZE = 32


class DequantScaleRoundingMode(Enum):
    ROUND_UP = 0    # scale = 2^ceil(log2(max / max_q)): never clips the group maximum
    ROUND_DOWN = 1  # scale = 2^floor(log2(max / largest power of two <= max_q)): OCP rule


def _as_3d(t: torch.Tensor, axis: int):
    """View of `t` as [nb, L, nr] with the axis in the middle, or None when the outer
    axes cannot be merged without a copy."""
    L = t.shape[axis]
    nb = 1
    for s in t.shape[:axis]:
        nb *= s
    nr = 1
    for s in t.shape[axis + 1:]:
        nr *= s

    def merged_stride(dims):
        dims = [d for d in dims if t.shape[d] != 1]
        if not dims:
            return 0
        for a, b in zip(dims[:-1], dims[1:]):
            if t.stride(a) != t.stride(b) * t.shape[b]:
                return None
        return t.stride(dims[-1])

    sb = merged_stride(range(0, axis))
    sr = merged_stride(range(axis + 1, t.ndim))
    if sb is None or sr is None:
        return None
    return nb, L, nr, sb, t.stride(axis), sr


def downcast_to_mxfp(x, out_dtype, axis: int, scale_dtype: torch.dtype = torch.uint8,
                     microblock_size: int = MXFP_BLOCK_SIZE,
                     DEQUANT_SCALE_ROUNDING_MODE: DequantScaleRoundingMode = DequantScaleRoundingMode.ROUND_UP):
    """Quantises `x` along `axis` in groups of 32: returns (values, scales) as torch
    tensors whose storage is contiguous along `axis`; FP4 values pack two codes per
    byte along it (even index in the low nibble)."""
    if isinstance(x, Tensor):
        x = x.storage.data
    assert scale_dtype == torch.uint8 or scale_dtype == torch.float8_e4m3fn, f"Invalid scale dtype {scale_dtype=}"
    assert x.shape[axis] % microblock_size == 0, \
        f"axis dim must be divisible by {microblock_size}. Got {x.shape[axis]}"
    assert -x.ndim <= axis < x.ndim, f"Invalid axis {axis=}"
    assert out_dtype in (torch.uint8, FP4, torch.float8_e4m3fn, torch.float8_e5m2), f"Invalid output dtype {out_dtype=}"
    assert x.dtype in (torch.float32, torch.bfloat16, torch.float16), f"Invalid input tensor dtype {x.dtype}"
    if scale_dtype != torch.uint8 or microblock_size != MXFP_BLOCK_SIZE:
        raise NotImplementedError("only e8m0 scales per 32 elements are built for gfx950")
    _lib.require_gpu(x, "x")
    axis = axis % x.ndim
    layout = StridedLayout(major_dim=axis - x.ndim)
    L = x.shape[axis]
    is_fp4 = out_dtype in (torch.uint8, FP4)
    value_code = _lib.MXFP4 if is_fp4 else _lib.dtype_code(out_dtype)
    if not is_fp4 and x.numel() > 0 and x.stride(axis) != 1:
        # fp8 values are quantised by the kernel for a contiguous axis only: move it last, quantise, move it back
        vt, st = downcast_to_mxfp(x.transpose(axis, -1).contiguous(), out_dtype, -1, scale_dtype, microblock_size,
                                  DEQUANT_SCALE_ROUNDING_MODE)
        return vt.transpose(axis, -1), st.transpose(axis, -1)
    y_value = empty(list(x.shape), FP4 if is_fp4 else torch_dtype_to_dtype(out_dtype), x.device, layout)
    scale_shape = [*x.shape[:axis], L // microblock_size, *x.shape[axis + 1:]]
    y_scale = empty(scale_shape, UINT8, x.device, layout)
    if x.numel() > 0:
        view = _as_3d(x, axis)
        if view is None or (view[4] != 1 and view[5] != 1 and view[2] != 1):
            x = x.contiguous()
            view = _as_3d(x, axis)
        nb, L, nr, sb, sl, sr = view
        if nr == 1:
            sr = 1 if sl != 1 else 0
        v, s = y_value.storage.data, y_scale.storage.data
        vv, sv = _as_3d(v, axis), _as_3d(s, axis)
        if vv is None or sv is None:
            # output axes after `axis` are not mergeable: quantise with the axis moved last, then re-lay
            vt, st = downcast_to_mxfp(x.transpose(axis, -1), out_dtype, -1, scale_dtype, microblock_size,
                                      DEQUANT_SCALE_ROUNDING_MODE)
            v.copy_(vt.transpose(axis, -1))
            s.copy_(st.transpose(axis, -1))
            return v, s
        rc = _lib.lib().tamd_downcast_mxfp(_lib.ptr(x), _lib.dtype_code(x.dtype), nb, L, nr, sb, sl, sr,
                                           _lib.ptr(v), value_code, vv[3], vv[5], _lib.ptr(s), sv[3], sv[5],
                                           DEQUANT_SCALE_ROUNDING_MODE.value, _lib.stream_ptr(x.device))
        _lib.check(rc, "downcast_to_mxfp")
    return y_value.storage.data, y_scale.storage.data


def upcast_from_mxfp(tensor: torch.Tensor, scale: torch.Tensor, target_dtype: torch.dtype, axis: int,
                     tensor_scale=None):
    """Inverse of downcast_to_mxfp; the result is contiguous in the logical axis order."""
    ndim = tensor.ndim
    assert -ndim <= axis < ndim, f"Invalid axis {axis=}"
    axis = axis % ndim
    assert tensor.ndim == scale.ndim, \
        f"Weight and scale must have the same number of dimensions. Got {tensor.ndim=} and {scale.ndim=}"
    assert tensor.dtype in {torch.uint8, torch.float8_e5m2, torch.float8_e4m3fn}, f"Invalid tensor dtype {tensor.dtype=}"
    assert scale.dtype == torch.uint8 or scale.dtype == torch.float8_e4m3fn, f"Invalid scale dtype {scale.dtype=}"
    assert target_dtype in (torch.float16, torch.bfloat16, torch.float32), f"Invalid output dtype {target_dtype=}"
    if scale.dtype != torch.uint8:
        raise NotImplementedError("only e8m0 scales are built for gfx950")
    _lib.require_gpu(tensor, "tensor")
    is_fp4 = tensor.dtype == torch.uint8
    value_code = _lib.MXFP4 if is_fp4 else _lib.dtype_code(tensor.dtype)
    L = tensor.shape[axis] * (2 if is_fp4 else 1)
    if not is_fp4 and axis != ndim - 1:
        # fp8 values are dequantised by the kernel into a contiguous axis only
        out = upcast_from_mxfp(tensor.transpose(axis, -1).contiguous(), scale.transpose(axis, -1).contiguous(),
                               target_dtype, -1, None).transpose(axis, -1).contiguous()
        if tensor_scale is not None:
            shape = (1, ) * out.ndim if tensor_scale.numel() == 1 else (*tensor_scale.shape[:axis], 1,
                                                                        *tensor_scale.shape[axis:])
            out = out * tensor_scale.to(device=out.device).reshape(shape)
        return out
    out_shape = [*tensor.shape[:axis], L, *tensor.shape[axis + 1:]]
    out = torch.empty(out_shape, dtype=target_dtype, device=tensor.device)
    if out.numel() > 0:
        if tensor.stride(axis) != 1 or _as_3d(tensor, axis) is None:
            tensor = tensor.movedim(axis, -1).contiguous().movedim(-1, axis)  # unit stride along axis, the rest in order
        if scale.stride(axis) != 1 or _as_3d(scale, axis) is None:
            scale = scale.movedim(axis, -1).contiguous().movedim(-1, axis)
        vv, sv, ov = _as_3d(tensor, axis), _as_3d(scale, axis), _as_3d(out, axis)
        nb, _, nr = ov[0], ov[1], ov[2]
        dsl, dsr = ov[4], ov[5]
        if nr == 1:
            dsl, dsr = 1, 0
        rc = _lib.lib().tamd_upcast_mxfp(_lib.ptr(tensor), value_code, vv[3], vv[5], _lib.ptr(scale), sv[3], sv[5],
                                         _lib.ptr(out), _lib.dtype_code(target_dtype), nb, L, nr, ov[3], dsl, dsr,
                                         _lib.stream_ptr(tensor.device))
        _lib.check(rc, "upcast_from_mxfp")
    if tensor_scale is not None:
        shape = (1, ) * out.ndim if tensor_scale.numel() == 1 else (*tensor_scale.shape[:axis], 1,
                                                                    *tensor_scale.shape[axis:])
        out = out * tensor_scale.to(device=out.device).reshape(shape)
    return out
