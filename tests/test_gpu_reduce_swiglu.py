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
    rv, rs = MR.reduce_mx_ref(xv, xs, dim, mask=mask, scale=None if scale is None else (scale * 0.75 if use_flex else scale),
                              x_flex_scale=None)
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
