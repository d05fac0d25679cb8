"""GPU parity: seeded sweeps over shapes of routing, MXFP quantise / dequantise and reduce that the hand-picked cases
of the other files do not enumerate (odd sizes, every axis, every value type), each against the CPU oracle: integer
and byte results bit for bit, sums within the tolerance written in the test."""
import os
import random

import pytest
import torch

from oracle import matmul_ref as MR
from oracle import routing_ref as R
from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
from triton_amd.numerics_details.mxfp import DequantScaleRoundingMode, downcast_to_mxfp, upcast_from_mxfp
from triton_amd.reduce import reduce
from triton_amd.routing import routing

pytestmark = pytest.mark.gpu
CASES = range(int(os.environ.get("TAMD_SWEEP_CASES", "40")))  # TAMD_SWEEP_CASES widens the sweeps for exploration


@pytest.mark.parametrize("seed", CASES)
def test_sweep_routing(seed, device):
    rng = random.Random(2000 + seed)
    T = rng.choice([1, 2, 15, 16, 17, 63, 64, 65, 255, 300, 1000, 2049, 5000])
    E = rng.choice([1, 2, 3, 8, 31, 32, 33, 64, 100, 128, 129, 257, 500])
    k = rng.choice([k for k in (1, 2, 4, 8) if k <= E])
    ties = rng.random() < 0.4
    print("case", dict(seed=seed, T=T, E=E, k=k, ties=ties), flush=True)
    torch.manual_seed(seed)
    logits = torch.randn(T, E)
    if ties:
        logits = (logits * 2).round() / 2  # many exact ties: the lower column index must win
    out = routing(logits.to(device), k)
    ref = R.routing_ref(logits, k)
    assert torch.equal(out.indx.cpu().int(), ref["indx"])
    assert torch.equal(out.col_sum.cpu(), ref["col_sum"])
    assert torch.equal(out.scatter_indx.cpu(), ref["scatter_indx"])
    assert torch.equal(out.row_sorted_indx.cpu(), ref["row_sorted_indx"])
    assert torch.equal(out.gather_indx.cpu(), ref["gather_indx"])
    rm = out.ragged_metadata
    assert torch.equal(rm.slice_offs.cpu(), ref["ragged"].slice_offs)
    assert torch.equal(rm.block_offs_data.cpu(), ref["ragged"].block_offs_data)
    assert torch.equal(rm.block_schedule_data.cpu(), ref["ragged"].block_schedule_data)
    torch.testing.assert_close(out.vals.cpu(), ref["vals"], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("seed", CASES)
def test_sweep_mxfp(seed, device):
    rng = random.Random(3000 + seed)
    ndim = rng.choice([2, 3, 3, 4])
    axis = rng.randrange(ndim)
    shape = [rng.choice([1, 2, 3, 5, 8, 17, 40, 66]) for _ in range(ndim)]
    shape[axis] = 32 * rng.choice([1, 2, 3, 7, 16])
    vdt = rng.choice([torch.uint8, torch.uint8, torch.float8_e4m3fn, torch.float8_e5m2])
    src = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    dst = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    mode = rng.choice(list(DequantScaleRoundingMode))
    print("case", dict(seed=seed, shape=shape, axis=axis, vdt=vdt, src=src, dst=dst, mode=mode), flush=True)
    torch.manual_seed(seed)
    x = (torch.randn(shape) * torch.exp(torch.randn(shape) * 2)).to(src)
    x.view(-1)[::13] = 0
    rv, rs = downcast_to_mxfp_ref(x, vdt, axis, "up" if mode.value == 0 else "down")
    v, s = downcast_to_mxfp(x.to(device), vdt, axis, DEQUANT_SCALE_ROUNDING_MODE=mode)
    assert torch.equal(s.cpu(), rs), "scales differ"
    assert torch.equal(v.cpu().view(torch.uint8), rv.view(torch.uint8)), "values differ"
    back = upcast_from_mxfp(v, s, dst, axis)
    ref_back = upcast_from_mxfp_ref(rv, rs, dst, axis)
    assert back.dtype == dst and back.shape == ref_back.shape
    assert torch.equal(back.cpu().view(torch.int16 if dst.itemsize == 2 else torch.int32),
                       ref_back.view(torch.int16 if dst.itemsize == 2 else torch.int32)), "dequantised values differ"


@pytest.mark.parametrize("seed", CASES)
def test_sweep_reduce(seed, device):
    rng = random.Random(4000 + seed)
    ndim = rng.choice([2, 3, 3, 4])
    shape = [rng.choice([1, 2, 3, 4, 8, 33, 64, 100, 257]) for _ in range(ndim)]
    dim = rng.randrange(ndim)
    dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
    y_dtype = rng.choice([None, None, torch.float32]) if dtype != torch.float32 else rng.choice([None, torch.bfloat16, torch.float16])

    def operand_shape():
        # full, or broadcast (size 1) along a random subset of axes
        return [n if rng.random() < 0.6 else 1 for n in shape]

    mask_shape = operand_shape() if rng.random() < 0.6 else None
    scale_shape = operand_shape() if rng.random() < 0.5 else None
    print("case", dict(seed=seed, shape=shape, dim=dim, dtype=dtype, y_dtype=y_dtype, mask=mask_shape, scale=scale_shape), flush=True)
    torch.manual_seed(seed)
    x = torch.randn(shape).to(dtype)
    mask = None if mask_shape is None else torch.rand(mask_shape) > 0.3
    scale = None if scale_shape is None else torch.rand(scale_shape)
    y, _ = reduce(x.to(device), dim, mask=None if mask is None else mask.to(device),
                  scale=None if scale is None else scale.to(device), y_dtype=y_dtype)
    out_dtype = y_dtype or dtype
    # the oracle sums in float32 and rounds to the type of its input: fed the same values as float32 it returns
    # the unrounded sum, which is then rounded once to the output type
    ref = MR.reduce_ref(x.float(), dim, mask=mask, scale=scale).to(out_dtype)
    assert y.dtype == out_dtype and tuple(y.shape) == tuple(ref.shape)
    # sums of at most 257 terms of size ~1 in float32, then one rounding to the output type
    tol = dict(rtol=1e-2, atol=2e-2) if out_dtype != torch.float32 else dict(rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(y.cpu().float(), ref.float(), **tol)
