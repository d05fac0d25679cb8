"""GPU parity: top-k combine (reduce) and standalone SwiGLU vs the CPU oracle."""
import pytest
import torch

from oracle import matmul_ref as MR
from triton_amd.reduce import reduce
from triton_amd.swiglu import PrecisionConfig, swiglu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,dim", [((512, 4, 2880), 1), ((4, 300, 64), 0), ((37, 5, 33), 1), ((8, 16), 1), ((6, 7, 8), 2)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("mask_mode", [None, "full", "broadcast_last"])
def test_reduce(shape, dim, dtype, mask_mode, device):
    torch.manual_seed(0)
    x = torch.randn(shape).to(dtype)
    mask = None
    if mask_mode == "full":
        mask = torch.rand(shape) > 0.3
    elif mask_mode == "broadcast_last":
        mshape = list(shape)
        mshape[-1] = 1
        mask = torch.rand(mshape) > 0.3
    y, _ = reduce(x.to(device), dim, mask=None if mask is None else mask.to(device))
    ref = MR.reduce_ref(x, dim, mask=mask)
    tol = dict(rtol=1e-2, atol=1e-2) if dtype != torch.float32 else dict(rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(y.cpu().float(), ref.float(), **tol)


def test_reduce_scale(device):
    torch.manual_seed(1)
    x = torch.randn(64, 4, 256).to(torch.bfloat16)
    scale = torch.rand(64, 4, 1)
    y, _ = reduce(x.to(device), 1, scale=scale.to(device))
    ref = MR.reduce_ref(x, 1, scale=scale)
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("M,N", [(1311, 4352), (7, 30)])
@pytest.mark.parametrize("limit", [1e-2, 10.0, None])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_swiglu(M, N, limit, dtype, device):
    torch.manual_seed(2)
    x = torch.randn(M, N).to(dtype)
    out = swiglu(x.to(device), 0.5, PrecisionConfig(limit))
    ref = MR.swiglu_ref(x, 0.5, limit)
    tol = dict(rtol=1e-2, atol=1e-2) if dtype != torch.float32 else dict(rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol)


@pytest.mark.parametrize("shape,dim", [((64, 4, 256), 1), ((4, 40, 96), 0), ((37, 5, 64), 1)])
@pytest.mark.parametrize("mask_mode", [None, "broadcast_last"])
@pytest.mark.parametrize("use_scale,use_flex", [(False, False), (True, False), (True, True)])
def test_reduce_mxfp8_in_and_out(shape, dim, mask_mode, use_scale, use_flex, device):
    """Microscaled branch: fp8 values + e8m0 scales along the last axis in, the same out; bit-exact against the oracle
    (which adds in index order, as the kernel does)."""
    from oracle.mxfp_ref import downcast_to_mxfp_ref
    from triton_amd.numerics import InFlexData
    torch.manual_seed(0)
    x0 = torch.randn(shape) * torch.exp(torch.randn(shape[:-1] + (1, )))
    xv, xs = downcast_to_mxfp_ref(x0, torch.float8_e4m3fn, axis=-1)
    xv, xs = xv.contiguous(), xs.contiguous()
    mask = None
    if mask_mode == "broadcast_last":
        mask = torch.rand(shape[:-1] + (1, )) > 0.3
    sshape = [1] * len(shape)
    sshape[dim] = shape[dim]
    scale = torch.rand(sshape) + 0.5 if use_scale else None
    fscale = torch.tensor([0.75]) if use_flex else None
    yv, ys = reduce(xv.to(device), dim, mask=None if mask is None else mask.to(device),
                    scale=None if scale is None else scale.to(device), x_mxscale=xs.to(device),
                    x_flex=InFlexData(dtype=torch.float8_e4m3fn, scale=fscale.to(device)) if use_flex else InFlexData())
    rv, rs = MR.reduce_mx_ref(xv, xs, dim, mask=mask, scale=scale, x_flex_scale=fscale)
    assert yv.dtype == torch.float8_e4m3fn and torch.equal(ys.cpu(), rs)
    assert torch.equal(yv.cpu().view(torch.uint8), rv.contiguous().view(torch.uint8))


@pytest.mark.parametrize("shape,dim", [((8, 4096, 256), 1), ((2048, 40), 0), ((3, 1000, 7), 1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_reduce_long_axis(shape, dim, dtype, device):
    """A long reduced axis over few outputs is summed in chunks (float32 partial sums): same sum up to the order of
    the additions."""
    torch.manual_seed(0)
    x = torch.randn(shape).to(dtype)
    y, _ = reduce(x.to(device), dim)
    ref = MR.reduce_ref(x, dim)
    assert y.dtype == dtype and tuple(y.shape) == tuple(ref.shape)
    tol = dict(rtol=1e-2, atol=5e-1) if dtype != torch.float32 else dict(rtol=1e-4, atol=1e-3)
    torch.testing.assert_close(y.cpu().float(), ref.float(), **tol)


# ---------------------------------------------------------------------------- the general reduction
# after tests/test_reduce.py:41-120 of the reference (shapes scaled to what the CPU oracle sums in a second)

def _init_mask(mode, B, M, N):
    if mode == "none":
        return None
    shape = {"full": (B, M, N), "broadcast_b": (1, M, N), "broadcast_m": (B, 1, N), "broadcast_n": (B, M, 1)}[mode]
    return torch.rand(shape) > 0.3


@pytest.mark.parametrize("B,M,N,postprocess", [(31, 384, 96, None), (64, 31, 384, None), (48, 64, 311, None), (64, 64, 128, None),
                                               (64, 64, 128, "plus_ten"), (64, 64, 128, "swiglu"), (4, 4, 4, None), (3, 15, 25, None),
                                               (5, 999, 235, None), (15, 345, 78, "plus_ten")])
@pytest.mark.parametrize("dtype_str", ["float16", "bfloat16", "float32", "mxfloat8", "flexfloat8_e4m3fn", "flexfloat8_e5m2"])
@pytest.mark.parametrize("mask_mode", ["none", "full", "broadcast_b", "broadcast_m", "broadcast_n"])
@pytest.mark.parametrize("dim", [0, 1, 2])
def test_reduce_general(B, M, N, postprocess, dtype_str, mask_mode, dim, device):
    from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
    from triton_amd.numerics import InFlexData, OutFlexData
    from triton_amd.reduce import PostprocessFn, plus_a_reduce
    from triton_amd.specialize import FnSpecs
    from triton_amd.swiglu import swiglu_fn
    if mask_mode not in ("none", "full") and (B, M, N) not in ((64, 64, 128), (3, 15, 25), (48, 64, 311)):
        pytest.skip("broadcast masks are exercised on three of the shapes")
    torch.manual_seed(0)
    x = torch.randn(B, M, N)
    is_mx, is_flex = dtype_str.startswith("mx"), dtype_str.startswith("flex")
    xs = fscale = expected = None
    if is_mx:
        x, xs = downcast_to_mxfp_ref(x.to(torch.float16), torch.float8_e4m3fn, axis=-1)
        x, xs = x.contiguous(), xs.contiguous()
    elif is_flex:
        dt = getattr(torch, dtype_str.removeprefix("flex"))
        fscale, expected = torch.tensor([2.0]), torch.tensor([4.0])
        x = (x / fscale).to(dt)
    else:
        x = x.to(getattr(torch, dtype_str))
    mask = _init_mask(mask_mode, B, M, N)
    if dim == 2 and is_mx:
        with pytest.raises(ValueError):
            reduce(x.to(device), dim=dim, mask=None if mask is None else mask.to(device), x_mxscale=xs.to(device))
        return
    pp_tri, pp_ref = None, None
    if postprocess is not None:
        if dim == 2 or [B, M, N][2] % 2:
            pytest.skip("the post-processing functions pair up columns of the last axis")
        if postprocess == "plus_ten":
            pp_tri, pp_ref = PostprocessFn(FnSpecs("plus_a", plus_a_reduce, ("a", ), reduction_n=2), (10, )), ("plus_a", 10.0)
        else:
            pp_tri = PostprocessFn(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))
            pp_ref = ("swiglu", 1.702, 7.0)
    actual = torch.zeros(1, device=device)
    y, y_mx = reduce(x.to(device), dim=dim, mask=None if mask is None else mask.to(device),
                     x_mxscale=None if xs is None else xs.to(device),
                     x_flex=InFlexData(scale=fscale.to(device)) if is_flex else InFlexData(),
                     y_flex=OutFlexData(expected_scale=expected.to(device), actual_scale=actual) if is_flex else OutFlexData(),
                     postprocess_fn1=pp_tri)
    ry, ry_mx, ractual = MR.reduce_general_ref(x, dim, mask=mask, x_mxscale=xs, x_flex_scale=fscale, postprocess=pp_ref,
                                               y_expected_scale=expected, y_has_mx=is_mx)
    assert y.dtype == x.dtype and tuple(y.shape) == tuple(ry.shape)
    if is_mx:
        # bit-exact unless the post-processing function's transcendental differs in the last place
        if postprocess == "swiglu":
            a = upcast_from_mxfp_ref(y.cpu(), y_mx.cpu(), torch.float32, axis=-1)
            b = upcast_from_mxfp_ref(ry, ry_mx, torch.float32, axis=-1)
            torch.testing.assert_close(a, b, rtol=0.13, atol=1e-3)
        else:
            assert torch.equal(y_mx.cpu(), ry_mx)
            assert torch.equal(y.cpu().view(torch.uint8), ry.contiguous().view(torch.uint8))
        return
    assert y_mx is None
    if is_flex:
        torch.testing.assert_close(actual.cpu(), ractual, rtol=1e-6, atol=1e-30)
    if postprocess == "swiglu":
        torch.testing.assert_close(y.cpu().float(), ry.float(), rtol=0.13 if is_flex else 2e-3, atol=1e-3)
    else:
        # the same float32 additions in the same order, the same casts: bit for bit
        assert torch.equal(y.cpu().view(torch.uint8), ry.contiguous().view(torch.uint8))


@pytest.mark.parametrize("saturate", [False, True])
@pytest.mark.parametrize("y_dtype", [torch.float8_e4m3fn, torch.float8_e5m2, torch.float16])
def test_reduce_flex_output_saturation_and_global_scale(saturate, y_dtype, device):
    """Sums far beyond the output type's range: clamped when saturating, the type's overflow value otherwise; the global
    scale enters after the sum; the actual scale is the maximum before the division (flexpoint.py:137-188)."""
    from triton_amd.numerics import OutFlexData
    torch.manual_seed(1)
    x = torch.randn(40, 6, 96) * 300
    expected, gscale = torch.tensor([0.01]), torch.tensor([3.0])
    actual = torch.zeros(1, device=device)
    y, _ = reduce(x.to(device), dim=1, x_global_scale=gscale.to(device), y_dtype=y_dtype,
                  y_flex=OutFlexData(expected_scale=expected.to(device), actual_scale=actual), y_flex_saturate_inf=saturate)
    ry, _, ractual = MR.reduce_general_ref(x, 1, x_global_scale=gscale, y_dtype=y_dtype, y_expected_scale=expected,
                                           y_saturate_inf=saturate)
    a, b = y.cpu().float(), ry.float()
    assert torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(torch.nan_to_num(a), torch.nan_to_num(b))
    torch.testing.assert_close(actual.cpu(), ractual, rtol=1e-6, atol=0)
    if saturate:
        assert torch.isfinite(a).all()


def test_reduce_refuses_what_is_not_built(device):
    from triton_amd.reduce import PostprocessFn
    from triton_amd.specialize import FnSpecs
    x = torch.randn(4, 3, 64, device=device)
    with pytest.raises(NotImplementedError):
        reduce(x, 1, postprocess_fn1=PostprocessFn(FnSpecs("gelu", None, (), reduction_n=1), ()))
    with pytest.raises(NotImplementedError):
        reduce(x, 1, y_value_pack_factor=2, y_has_mx=True)


@pytest.mark.parametrize("shape,dim", [((512, 4, 2880), 1), ((3, 64, 4, 512), 2), ((5, 4, 100), 1), ((64, 7, 264), 1)])
@pytest.mark.parametrize("x_dtype", [torch.float8_e4m3fn, torch.float8_e5m2, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("y_dtype", [None, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("scales", ["none", "flex", "flex+global"])
def test_reduce_plain_sums_of_fp8_and_scaled_rows(shape, dim, x_dtype, y_dtype, scales, device):
    """The top-k combine of fp8 rows (and plain sums with only the scalar input scales): dense aligned shapes take the
    kernel variant that compiles nothing but the vector paths, (5, 4, 100) the general one; bit for bit against the
    index-order float32 sum of the oracle."""
    from triton_amd.numerics import InFlexData
    torch.manual_seed(3)
    x = torch.randn(shape).to(x_dtype)
    fscale = torch.tensor([0.5]) if scales != "none" else None
    gscale = torch.tensor([3.0]) if scales == "flex+global" else None
    y, y_mx = reduce(x.to(device), dim=dim, x_flex=InFlexData(scale=fscale.to(device)) if fscale is not None else InFlexData(),
                     x_global_scale=None if gscale is None else gscale.to(device), y_dtype=y_dtype)
    ry, _, _ = MR.reduce_general_ref(x, dim, x_flex_scale=fscale, x_global_scale=gscale, y_dtype=y_dtype)
    assert y_mx is None and y.dtype == (y_dtype or x_dtype) and tuple(y.shape) == tuple(ry.shape)
    assert torch.equal(y.cpu().view(torch.uint8), ry.contiguous().view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn])
@pytest.mark.parametrize("with_mask", [True, False])
def test_reduce_unpadded_batch_size(dtype, with_mask, device):
    """tests/test_reduce.py:156-176 of the reference: B, M, N = 7, 73, 257 reduced over B with a device-side count of 37
    rows; the rows past it keep what y held."""
    torch.manual_seed(0)
    B, M, N, unpadded, sentinel = 7, 73, 257, 37, -1234.0
    x = torch.randn(B, M, N).to(dtype)
    y_dtype = torch.float16 if dtype == torch.float8_e4m3fn else dtype
    mask = torch.ones((B, M, 1), dtype=torch.int8).expand(B, M, N) if with_mask else None
    y = torch.full((M, N), sentinel, dtype=y_dtype, device=device)
    got, _ = reduce(x.to(device), dim=0, mask=None if mask is None else mask.to(device), y=y, y_dtype=y_dtype,
                    unpadded_batch_size=torch.tensor(unpadded, device=device, dtype=torch.int32))
    want, _, _ = MR.reduce_general_ref(x, 0, y_dtype=y_dtype, unpadded_batch_size=torch.tensor(unpadded))
    assert got.data_ptr() == y.data_ptr()
    assert torch.equal(got[:unpadded].cpu().view(torch.uint8), want.contiguous().view(torch.uint8))
    assert torch.equal(got[unpadded:].cpu(), torch.full((M - unpadded, N), sentinel, dtype=y_dtype))
    # a count beyond the axis reduces every row; zero reduces none
    y2 = torch.full((M, N), sentinel, dtype=y_dtype, device=device)
    reduce(x.to(device), dim=0, y=y2, y_dtype=y_dtype, unpadded_batch_size=torch.tensor(10 ** 6, device=device, dtype=torch.int32))
    full, _, _ = MR.reduce_general_ref(x, 0, y_dtype=y_dtype)
    assert torch.equal(y2.cpu().view(torch.uint8), full.contiguous().view(torch.uint8))
    y3 = torch.full((M, N), sentinel, dtype=y_dtype, device=device)
    reduce(x.to(device), dim=0, y=y3, y_dtype=y_dtype, unpadded_batch_size=torch.tensor(0, device=device, dtype=torch.int32))
    assert torch.equal(y3.cpu(), torch.full((M, N), sentinel, dtype=y_dtype))


@pytest.mark.parametrize("R", [1, 4, 8, 9])
@pytest.mark.parametrize("shape_tail", [(2880, ), (33, )])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float8_e4m3fn])
def test_reduce_sign_of_zero_follows_the_reference_kernel(R, shape_tail, dtype, device):
    """Columns of -0.0: the first term starts the sum for an axis of at most 8 entries (reduce.py:137, 467-470 of the
    reference), so the result is -0.0; a longer axis starts from +0.0.  With a scale every term passes through
    fma(x, s, +0.0) and the result is +0.0; a masked first entry counts as +0.0."""
    x = torch.full((16, R, *shape_tail), -0.0).to(dtype)
    y_dtype = torch.bfloat16 if dtype == torch.float8_e4m3fn else dtype
    y, _ = reduce(x.to(device), 1, y_dtype=y_dtype)
    assert torch.signbit(y.float()).all().item() == (R <= 8)
    want, _, _ = MR.reduce_general_ref(x, 1, y_dtype=y_dtype)
    assert torch.equal(y.cpu().view(torch.uint8), want.contiguous().view(torch.uint8))
    ys, _ = reduce(x.to(device), 1, scale=torch.ones((1, R, 1), device=device), y_dtype=y_dtype)
    assert not torch.signbit(ys.float()).any().item()
    mask = torch.ones((16, R, 1), dtype=torch.bool)
    mask[::2, 0] = False
    ym, _ = reduce(x.to(device), 1, mask=mask.to(device), y_dtype=y_dtype)
    wm, _, _ = MR.reduce_general_ref(x, 1, mask=mask, y_dtype=y_dtype)
    assert torch.equal(ym.cpu().view(torch.uint8), wm.contiguous().view(torch.uint8))
