"""Reduction over one axis with every optional operand of the reference's `reduce` (reduce.py:1135-1157): mask and
scale (broadcastable), microscaled or flexpoint inputs, a pairwise post-processing function, flexpoint or
microscaled outputs.  The plain sum -- the top-k combine, y.view(T, k, N) -> sum over k -- has a kernel of its own."""
import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from .numerics import InFlexData, OutFlexData
from .specialize import FnSpecs

MXFP_BLOCK_SIZE = 32


@dataclass(frozen=True)
class PostprocessFn:
    """A function applied to the sums before they are stored (reduce.py:26-29 of the reference).  The reference
    splices Triton source; here `specs.name` selects a compiled variant: "swiglu" (fn_args = (alpha, limit): SwiGLU of
    interleaved gate / linear column pairs, what a split-K matmul finishes with) and "plus_a" (fn_args = (a, ):
    (x + a) summed over column pairs, the function of the reference's own test, tests/test_reduce.py:35-38)."""
    specs: FnSpecs = FnSpecs.default()
    fn_args: tuple = tuple()


def plus_a_reduce(*_args, **_kwargs):
    """Tag carried in FnSpecs("plus_a", plus_a_reduce, ("a", ), reduction_n=2); the variant is selected by name."""
    raise RuntimeError("plus_a_reduce is a tag for the compiled post-processing variant, not a callable")


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


def _scalar(t, what):
    if t is None:
        return None
    if t.numel() != 1 or t.dtype != torch.float32:
        raise NotImplementedError(f"{what}: one float32 value expected (per-batch scales are not built)")
    return t


def _postprocess_code(fn: Optional[PostprocessFn]):
    """(code, arg0, arg1, has_arg1, reduction_n) of a post-processing function."""
    if fn is None or fn.specs is None or fn.specs.name == "dflt":
        return _lib.PP_NONE, 0.0, 0.0, 0, 1
    named = dict(zip(fn.specs.fn_arg_names, fn.fn_args))
    if fn.specs.name == "swiglu":
        assert fn.specs.reduction_n == 2
        alpha = named.get("alpha", fn.fn_args[0])
        limit = named.get("limit", fn.fn_args[1] if len(fn.fn_args) > 1 else None)
        return _lib.PP_SWIGLU, float(alpha), float(limit) if limit is not None else 0.0, int(limit is not None), 2
    if fn.specs.name == "plus_a":
        assert fn.specs.reduction_n == 2
        return _lib.PP_PLUS_A_PAIRSUM, float(named.get("a", fn.fn_args[0])), 0.0, 0, 2
    raise NotImplementedError(f"post-processing function {fn.specs.name!r} is not built (swiglu and plus_a are)")


def reduce(x: torch.Tensor, dim: int, mask: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
           x_mxscale: Optional[torch.Tensor] = None, x_flex: Optional[InFlexData] = InFlexData(),
           x_global_scale: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None,
           y_dtype: Optional[torch.dtype] = None, y_flex: Optional[OutFlexData] = OutFlexData(),
           y_flex_saturate_inf: bool = False, y_has_mx: Optional[bool] = None, y_mx_scale_dtype=None,
           y_microblock_size: int = MXFP_BLOCK_SIZE, y_value_pack_factor: int = 1,
           postprocess_fn1: Optional[PostprocessFn] = None, postprocess_fn2: Optional[PostprocessFn] = None,
           unpadded_batch_size=None):
    """Returns (y, y_mxscale).  y = postprocess(sum over `dim` of where(mask, x * scale, 0)), accumulated in float32 in
    index order; then the output's flexpoint scales or its MXFP8 quantisation along the last axis (when the input is
    microscaled, as in the reference, reduce.py:1185-1206); cast to y_dtype (default x.dtype)."""
    if unpadded_batch_size is not None:
        # a device-side count of the rows of the first kept axis that hold data (reduce.py:694-695, 550-555): the rest
        # of y is left as it is.  Read by the kernel, never on the host.
        assert unpadded_batch_size.numel() == 1, "unpadded_batch_size is a single-element tensor"
        _lib.require_gpu(unpadded_batch_size, "unpadded_batch_size")
        if unpadded_batch_size.dtype != torch.int32:
            unpadded_batch_size = unpadded_batch_size.to(torch.int32)
    if postprocess_fn2 is not None and postprocess_fn2.specs.name != "dflt":
        raise NotImplementedError("a second post-processing function is not built")
    if y_value_pack_factor != 1 or y_microblock_size != MXFP_BLOCK_SIZE:
        raise NotImplementedError("microscaled outputs are built as float8_e4m3fn values with one e8m0 byte per 32")
    _lib.require_gpu(x, "x")
    dim = dim % x.ndim
    if x_mxscale is not None and dim == x.ndim - 1:
        raise ValueError("reduction over the microscaled dimension is not supported")
    pp, pp0, pp1, pp_has1, rn = _postprocess_code(postprocess_fn1)
    if x_flex is not None:
        x = x_flex.reinterpret(x)
    x_flex_scale = _scalar(getattr(x_flex, "scale", None), "x_flex.scale")
    x_global_scale = _scalar(x_global_scale, "x_global_scale")
    y_expected = _scalar(getattr(y_flex, "expected_scale", None), "y_flex.expected_scale")
    y_actual = _scalar(getattr(y_flex, "actual_scale", None), "y_flex.actual_scale")
    if getattr(y_flex, "checksum_scale", None) is not None:
        raise NotImplementedError("flexpoint checksum is not built")
    if y_has_mx is None:
        y_has_mx = x_mxscale is not None
    if y_has_mx and y_actual is not None:
        raise NotImplementedError("a microscaled output keeps no flexpoint actual scale (reduce.py:480-484)")
    R = x.shape[dim]
    if unpadded_batch_size is not None and x.ndim != 3:
        raise NotImplementedError("unpadded_batch_size is built for 3-D inputs (the rows of the first kept axis)")
    if x.ndim == 3:
        # the reference's view (reduce.py:732-747): the two axes that stay are (S0, S1) with the strides they have
        d0, d1 = [d for d in range(3) if d != dim]
        lead, tail = x.shape[d0], x.shape[d1]
        x3 = x.permute(d0, dim, d1)

        def to3(t):
            if t is None:
                return None
            assert t.ndim == 3, "mask / scale must have the rank of x"
            return t.permute(d0, dim, d1)
    else:
        # any other rank (not in the reference): the axes before and after `dim` are merged, which needs a dense x
        lead = 1
        for n in x.shape[:dim]:
            lead *= n
        tail = 1
        for n in x.shape[dim + 1:]:
            tail *= n
        if (x_mxscale is not None or rn > 1 or y_has_mx) and tail != x.shape[-1]:
            raise NotImplementedError("microscaled / post-processed reductions of tensors that are not 3-D keep the last "
                                      "axis whole: reduce the axis before it")
        if not x.is_contiguous():
            x = x.contiguous()
        x3 = x.view(lead, R, tail)

        def to3(t):
            if t is None:
                return None
            assert t.ndim == x.ndim
            lead_t = 1
            for n in t.shape[:dim]:
                lead_t *= n
            tail_t = 1
            for n in t.shape[dim + 1:]:
                tail_t *= n
            if lead_t not in (1, lead) or tail_t not in (1, tail):
                t = t.expand(x.shape)
                lead_t, tail_t = lead, tail
            return t.reshape(lead_t, t.shape[dim], tail_t)

    assert tail % rn == 0, f"the post-processing function pairs up columns: {tail} is odd"
    out_shape = [*x.shape[:dim], *x.shape[dim + 1:]]
    out_shape[-1] //= rn
    if y_has_mx:
        y_dtype = y_dtype or torch.float8_e4m3fn
        if y_dtype != torch.float8_e4m3fn or y_mx_scale_dtype not in (None, torch.uint8):
            raise NotImplementedError("microscaled outputs are built as float8_e4m3fn values with e8m0 (uint8) scales")
    y_dtype = y_dtype or x.dtype
    plain = (x_mxscale is None and x_flex_scale is None and x_global_scale is None and pp == _lib.PP_NONE and not y_has_mx
             and y_expected is None and y_actual is None and x.dtype.itemsize > 1 and y_dtype.itemsize > 1
             and unpadded_batch_size is None)
    if plain and mask is None and scale is None and y is None and R >= 512 and lead * tail <= (1 << 18) and x.is_contiguous():
        # a long axis over few outputs: a thread of the kernel walks the whole axis, so it is cut into chunks that
        # are summed side by side (float32 partial sums), then the chunks are summed
        # (more than 8 chunks: the second sum then starts from +0.0 like the one long sum it stands for)
        chunks = next((c for c in (64, 32, 16) if R % c == 0), 0)
        if chunks:
            lead_c = 1
            for n in x.shape[:dim]:
                lead_c *= n
            part, _ = reduce(x.view(lead_c, chunks, R // chunks, -1), 2, y_dtype=torch.float32)
            out, _ = reduce(part, 1, y_dtype=y_dtype)
            return out.view(out_shape), None
    mask3, scale3 = to3(mask), to3(scale)
    if mask3 is not None:
        mask3 = mask3.to(torch.bool).view(torch.uint8) if mask3.dtype != torch.uint8 else mask3
    if scale3 is not None and scale3.dtype != torch.float32:
        scale3 = scale3.to(torch.float32)
    if y is None:
        y = torch.empty(out_shape, dtype=y_dtype, device=x.device)
    else:
        assert list(y.shape) == out_shape and y.is_contiguous() and y.dtype == y_dtype
    y2 = y.view(lead, tail // rn)
    ms, ss = _bstrides(mask3, x3.shape), _bstrides(scale3, x3.shape)
    if plain:
        rc = _lib.lib().tamd_reduce(_lib.ptr(x3), _lib.dtype_code(x.dtype), lead, R, tail, x3.stride(0), x3.stride(1),
                                    x3.stride(2), _lib.ptr(mask3), *ms, _lib.ptr(scale3), *ss, _lib.ptr(y2),
                                    _lib.dtype_code(y_dtype), y2.stride(0), y2.stride(1), _lib.stream_ptr(x.device))
        _lib.check(rc, "reduce")
        return y, None
    a = _lib.ReduceArgs()
    a.x, a.x_dtype, a.S0, a.R, a.S1 = x3.data_ptr(), _lib.dtype_code(x.dtype), lead, R, tail
    a.xs0, a.xsr, a.xs1 = x3.stride()
    if x_mxscale is not None:
        assert x_mxscale.dtype == torch.uint8 and x_mxscale.ndim == x.ndim
        want = [*x.shape[:-1], -(-x.shape[-1] // MXFP_BLOCK_SIZE)]
        assert list(x_mxscale.shape) == want, f"x_mxscale shape {tuple(x_mxscale.shape)} != {tuple(want)}"
        xm = x_mxscale.permute(d0, dim, d1) if x.ndim == 3 else x_mxscale.contiguous().view(lead, R, -1)
        a.x_mx_scale = xm.data_ptr()
        a.xms0, a.xmsr, a.xms1 = xm.stride()
    a.x_flex_scale = None if x_flex_scale is None else x_flex_scale.data_ptr()
    a.x_global_scale = None if x_global_scale is None else x_global_scale.data_ptr()
    if mask3 is not None:
        a.mask = mask3.data_ptr()
        a.ms0, a.msr, a.ms1 = ms
    if scale3 is not None:
        a.scale = scale3.data_ptr()
        a.ss0, a.ssr, a.ss1 = ss
    a.postprocess, a.pp_arg0, a.pp_arg1, a.pp_has_arg1 = pp, pp0, pp1, pp_has1
    a.y, a.y_dtype = y2.data_ptr(), _lib.dtype_code(y_dtype)
    a.ys0, a.ys1 = y2.stride(0), y2.stride(1)
    a.y_expected_scale = None if y_expected is None else y_expected.data_ptr()
    a.y_actual_scale = None if y_actual is None else y_actual.data_ptr()
    a.y_saturate_inf = int(bool(y_flex_saturate_inf))
    a.unpadded_batch_size = None if unpadded_batch_size is None else unpadded_batch_size.data_ptr()
    y_mx = None
    if y_has_mx:
        y_mx = torch.empty([*out_shape[:-1], -(-out_shape[-1] // MXFP_BLOCK_SIZE)], dtype=torch.uint8, device=x.device)
        ym2 = y_mx.view(lead, -1)
        a.y_mx_scale = ym2.data_ptr()
        a.yms0, a.yms1 = ym2.stride(0), ym2.stride(1)
    rc = _lib.lib().tamd_reduce_ex(ctypes.byref(a), _lib.stream_ptr(x.device))
    _lib.check(rc, "reduce")
    return y, y_mx
