"""CPU oracle: grouped matmul, SwiGLU and the top-k combine.  Test infrastructure, never shipped.

Restates, with torch-CPU float32 arithmetic:
  matmul_ref   matmul.py:823-914 (matmul_torch) + :755-800 (apply_precision)
  swiglu_ref   swiglu.py:89-100 (swiglu_torch)
  reduce_ref   reduce.py:1173-1206 (reduce_torch), sum/mask/scale part
"""
import torch

from .mxfp_ref import upcast_from_mxfp_ref


def dequant_operand(t: torch.Tensor, mx_scale, flex_scale, mx_axis: int):
    """apply_precision (matmul.py:755-800): an mx operand is dequantised to
    bfloat16 (:772-778, 788-794); a flex (per-tensor scaled fp8) operand becomes
    float32 value*scale (:761-764); anything else is used as is."""
    if mx_scale is not None:
        return upcast_from_mxfp_ref(t, mx_scale, torch.bfloat16, axis=mx_axis)
    if flex_scale is not None:
        return t.to(torch.float32) * flex_scale.to(torch.float32)
    return t.clone()


def matmul_ref(a, b, bias, slice_sizes=None, gather_indx=None, scatter_indx=None,
               a_mx_scale=None, b_mx_scale=None, a_flex_scale=None, b_flex_scale=None,
               betas=None, gammas=None, out_scale=None, out_alpha=None, fused_swiglu=None):
    """y[rows of slice e] = (a[gather] @ deq(b[e])) + bias[e]*beta, times gamma,
    computed in float32 and stored in the dtype of the dequantised `a`
    (matmul.py:887-902); rows are then placed at scatter_indx (-1 drops the row,
    :905-910); the result is divided by out_scale when given (:914).

    fused_swiglu=(alpha, limit) applies the activation to the float32 result
    before gamma and before the cast, the order of the reference's GPU kernel
    (matmul_details/_matmul.py:540-559); without it the caller applies
    swiglu_ref to the rounded output, the order of the reference's test
    (tests/test_matmul.py:599-600).  out_alpha multiplies after the bias (:548-550).

    a: [M, K] (or [B, M, K] batched); b: [E, K, N] / [K, N], mxfp4 weights as
    packed uint8 [E, K/2, N] with b_mx_scale uint8 [E, K/32, N].
    slice_sizes: int32 [E] rows per expert in expert-sorted order (ragged M).
    """
    a = dequant_operand(a, a_mx_scale, a_flex_scale, a.ndim - 1)
    b = dequant_operand(b, b_mx_scale, b_flex_scale, b.ndim - 2)
    batched = a.ndim == 3
    if bias is not None and bias.ndim == 1:
        bias = bias[None]
    if b.ndim == 2:
        b = b[None]
    if a.ndim == 2:
        a = a[None]
    if slice_sizes is not None and not batched:
        offs = [0]
        for s in slice_sizes.tolist():
            offs.append(offs[-1] + int(s))
        spans = list(zip(offs[:-1], offs[1:]))
    else:
        spans = [(0, a.shape[1])] * b.shape[0]
    n_rows = a.shape[1] if gather_indx is None else gather_indx.shape[0]
    n_out = b.shape[-1] // 2 if fused_swiglu is not None else b.shape[-1]
    y = torch.zeros((a.shape[0], n_rows, n_out), dtype=a.dtype)
    for e, (lo, hi) in enumerate(spans):
        rows = torch.arange(lo, hi) if gather_indx is None else gather_indx[lo:hi].long()
        z = e if batched else 0
        out = a[z, rows, :].to(torch.float32) @ b[e].to(torch.float32)
        if bias is not None:
            bb = bias[e].to(torch.float32)
            out = out + (bb if betas is None else bb * betas[lo:hi, None].to(torch.float32))
        if out_alpha is not None:
            out = out * out_alpha
        if fused_swiglu is not None:
            out = swiglu_ref(out, fused_swiglu[0], fused_swiglu[1])
        if gammas is not None:
            out = out * gammas[lo:hi, None].to(torch.float32)
        y[z, lo:hi, :] = out.to(y.dtype)
    if not batched:
        y = y[0]
    if scatter_indx is not None:
        out = torch.zeros((scatter_indx.shape[0], y.shape[-1]), dtype=y.dtype)
        keep = scatter_indx != -1
        out[scatter_indx[keep].long()] = y[keep]
        y = out
    if out_scale is not None:
        y = y / out_scale
    return y


def actual_scale_ref(y: torch.Tensor, out_dtype) -> torch.Tensor:
    """max|y| / max_finite(out_dtype): what a flexpoint output records as its actual scale
    (compute_actual_scale, matmul.py:812-821 of the reference)."""
    return (y.float().abs().max() / torch.finfo(out_dtype).max).reshape(1)


def swiglu_ref(a: torch.Tensor, alpha: float, limit):
    """Interleaved SwiGLU, swiglu.py:89-100: gate = even columns clamped from
    above, linear = odd columns clamped to [-limit, limit];
    out = gate*sigmoid(alpha*gate) * (linear + 1), evaluated in float32."""
    dt = a.dtype
    a = a.to(torch.float32)
    g = a[..., 0::2]
    l = a[..., 1::2]
    if limit is not None:
        g = g.clamp(max=limit)
        l = l.clamp(min=-limit, max=limit)
    return ((g * torch.sigmoid(alpha * g)) * (l + 1)).to(dt)


def reduce_ref(x: torch.Tensor, dim: int, mask=None, scale=None):
    """sum over `dim` of where(mask, x*scale, 0) in float32, cast back to
    x.dtype; reduce.py:1179-1206 without the mx / flex branches."""
    xf = x.to(torch.float32)
    if scale is not None:
        xf = xf * scale.to(torch.float32)
    if mask is not None:
        xf = torch.where(mask.to(torch.bool), xf, torch.zeros((), dtype=torch.float32))
    return xf.sum(dim=dim).to(x.dtype)


def reduce_mx_ref(x: torch.Tensor, x_mxscale: torch.Tensor, dim: int, mask=None, scale=None, x_flex_scale=None):
    """The microscaled branch of reduce_torch (reduce.py:1185-1206): dequantise x (fp8 values, e8m0 scales along the
    last axis) to float32, masked / scaled sum over `dim`, quantise the float32 result to MXFP8 along the last axis.
    The sum runs in index order r = 0, 1, ... (one float32 addition per step), which fixes the rounding the GPU kernel
    has to reproduce.  Returns (values float8_e4m3fn, scales uint8)."""
    from .mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
    xf = upcast_from_mxfp_ref(x, x_mxscale, torch.float32, axis=-1)
    if x_flex_scale is not None:
        xf = xf * x_flex_scale.to(torch.float32)
    if scale is not None:
        xf = xf * scale.to(torch.float32)
    if mask is not None:
        xf = torch.where(mask.to(torch.bool), xf, torch.zeros((), dtype=torch.float32))
    dim = dim % xf.ndim
    acc = torch.zeros([n for i, n in enumerate(xf.shape) if i != dim], dtype=torch.float32)
    for r in range(xf.shape[dim]):
        acc = acc + xf.select(dim, r)
    return downcast_to_mxfp_ref(acc, torch.float8_e4m3fn, axis=-1)


def _index_order_sum(xf: torch.Tensor, dim: int) -> torch.Tensor:
    """float32 sum over `dim` in index order, one addition per step, started as the reference's kernel starts it
    (reduce.py:137 `use_static_loop = K <= 8`, :423-424, :467-470): for an axis of at most 8 entries the first term IS
    the initial value (so a column of -0.0 stays -0.0), longer axes start from +0.0."""
    n = xf.shape[dim]
    out_shape = [m for i, m in enumerate(xf.shape) if i != dim]
    if n == 0:
        return torch.zeros(out_shape, dtype=torch.float32)
    if n <= 8:
        acc = xf.select(dim, 0).clone()
        first = 1
    else:
        acc = torch.zeros(out_shape, dtype=torch.float32)
        first = 0
    for r in range(first, n):
        acc = acc + xf.select(dim, r)
    return acc


_MAX_FINITE = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0, torch.float16: 65504.0,
               torch.bfloat16: 3.3895313892515355e38, torch.float32: 3.4028234663852886e38}


def reduce_general_ref(x: torch.Tensor, dim: int, mask=None, scale=None, x_mxscale=None, x_flex_scale=None,
                       x_global_scale=None, postprocess=None, y_dtype=None, y_expected_scale=None,
                       y_saturate_inf: bool = False, y_has_mx: bool = False, unpadded_batch_size=None):
    """reduce_torch (reduce.py:1179-1210 of the reference) together with the operands only its kernel has
    (_reduce_forward_inner, reduce.py:441-492): the order of the factors of a term ((x * 2^e) * x_flex_scale) * scale,
    x_global_scale after the post-processing function, the flexpoint output as float_to_flex computes it
    (numerics_details/flexpoint.py:137-188: actual scale = max|y| / max_finite + 1e-30, y * (1 / expected), clamp when
    saturating).  Built from pieces that are pinned on their own -- upcast_from_mxfp_ref, swiglu_ref,
    downcast_to_mxfp_ref, torch's casts -- around an explicit index-order float32 sum.

    postprocess: None, ("swiglu", alpha, limit) or ("plus_a", a).  unpadded_batch_size: only that many entries of the
    first kept axis are reduced (reduce.py:550-555, 694-695; the kernel leaves the other rows of y alone), and only
    they are returned.  Returns (y, y_mxscale or None, actual_scale)."""
    from .mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
    y_dtype = y_dtype or x.dtype
    if unpadded_batch_size is not None:
        d0 = [d for d in range(x.ndim) if d != dim % x.ndim][0]
        n = int(unpadded_batch_size)
        narrow = lambda t: None if t is None else (t.narrow(d0, 0, n) if t.shape[d0] != 1 else t)
        x, mask, scale, x_mxscale = narrow(x), narrow(mask), narrow(scale), narrow(x_mxscale)
    xf = upcast_from_mxfp_ref(x, x_mxscale, torch.float32, axis=-1) if x_mxscale is not None else x.to(torch.float32)
    if x_flex_scale is not None:
        xf = xf * x_flex_scale.to(torch.float32)
    if scale is not None:
        xf = xf * scale.to(torch.float32) + torch.zeros((), dtype=torch.float32)  # tl.fma(x, s, 0.0), reduce.py:466
    if mask is not None:
        xf = torch.where(mask.to(torch.bool), xf, torch.zeros((), dtype=torch.float32))
    dim = dim % xf.ndim
    acc = _index_order_sum(xf, dim)
    if postprocess is not None:
        if postprocess[0] == "swiglu":
            acc = swiglu_ref(acc, postprocess[1], postprocess[2])
        elif postprocess[0] == "plus_a":
            t = acc + torch.tensor(postprocess[1], dtype=torch.float32)
            acc = t[..., 0::2] + t[..., 1::2]
        else:
            raise ValueError(postprocess[0])
    if x_global_scale is not None:
        acc = acc * x_global_scale.to(torch.float32)
    max_finite = _MAX_FINITE[torch.float8_e4m3fn if y_has_mx else y_dtype]
    absmax = acc.abs().max() if acc.numel() else torch.zeros(())
    absmax = torch.where(torch.isnan(absmax), torch.tensor(float("inf")), absmax)
    actual = (absmax * torch.tensor(1.0 / max_finite, dtype=torch.float32) + torch.tensor(1.0e-30, dtype=torch.float32)).reshape(1)
    if y_expected_scale is not None:
        acc = acc * (torch.ones((), dtype=torch.float32) / y_expected_scale.to(torch.float32))
        if y_saturate_inf and not y_has_mx:
            acc = acc.clamp(-max_finite, max_finite)
    if y_has_mx:
        v, s = downcast_to_mxfp_ref(acc, torch.float8_e4m3fn, axis=-1)
        return v, s, actual
    return acc.to(y_dtype), None, actual
