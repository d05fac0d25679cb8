"""GPU parity: downcast_to_mxfp / upcast_from_mxfp through the C ABI vs the CPU oracle (bit-exact)."""
import pytest
import torch

from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
from triton_amd.numerics_details.mxfp import DequantScaleRoundingMode, downcast_to_mxfp, upcast_from_mxfp

pytestmark = pytest.mark.gpu


def _check_quant(x_cpu, axis, device, mode=DequantScaleRoundingMode.ROUND_UP):
    ref_v, ref_s = downcast_to_mxfp_ref(x_cpu, torch.uint8, axis, "up" if mode.value == 0 else "down")
    v, s = downcast_to_mxfp(x_cpu.to(device), torch.uint8, axis, DEQUANT_SCALE_ROUNDING_MODE=mode)
    assert v.stride(axis) == 1 or v.shape[axis] == 1
    assert s.stride(axis) == 1 or s.shape[axis] == 1
    assert torch.equal(s.cpu(), ref_s), "scales differ"
    assert torch.equal(v.cpu(), ref_v), "codes differ"
    return v, s, ref_v, ref_s


@pytest.mark.parametrize("shape,axis", [((256, 2048), 1), ((2048, 512), 0), ((3, 96, 200), 1), ((3, 96, 224), -1),
                                        ((5, 64, 33), 1), ((7, 32), 1), ((32, 7), 0), ((2, 3, 64, 40), 2),
                                        ((4, 64, 6, 10), 1), ((64, 5, 8), 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_downcast_matches_oracle(shape, axis, dtype, device):
    torch.manual_seed(0)
    if shape[axis] % 32 != 0:
        pytest.skip("axis not divisible by 32")
    x = (torch.randn(shape) * torch.exp(torch.randn(shape) * 2)).to(dtype)
    x.view(-1)[::17] = 0
    _check_quant(x, axis, device)


@pytest.mark.parametrize("mode", list(DequantScaleRoundingMode))
def test_rounding_modes(mode, device):
    torch.manual_seed(1)
    x = torch.randn(64, 256) * 10
    _check_quant(x, 1, device, mode)


def test_config1_weight_roundtrip(device):
    """BASELINE config 1: W fp32 [2048, 4096] ~N(0, 0.02) quantised along K."""
    torch.manual_seed(0)
    w = torch.randn(2048, 4096) * 0.02
    v, s, ref_v, ref_s = _check_quant(w, 0, device)
    assert tuple(v.shape) == (1024, 4096) and v.stride() == (1, 1024)
    assert tuple(s.shape) == (64, 4096) and s.stride() == (1, 64)
    for dt in (torch.bfloat16, torch.float32, torch.float16):
        out = upcast_from_mxfp(v, s, dt, axis=0)
        ref = upcast_from_mxfp_ref(ref_v, ref_s, dt, axis=0)
        assert out.is_contiguous()
        assert torch.equal(out.cpu().view(torch.uint8), ref.contiguous().view(torch.uint8))


@pytest.mark.parametrize("shape,axis", [((128, 512), 1), ((512, 128), 0), ((4, 64, 72), 1), ((4, 72, 64), 2), ((9, 32, 5), 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_upcast_matches_oracle(shape, axis, dtype, device):
    torch.manual_seed(2)
    x = torch.randn(shape) * 3
    ref_v, ref_s = downcast_to_mxfp_ref(x, torch.uint8, axis)
    # every scale byte, including 0 and 0xFF
    ref_s = ref_s.contiguous()
    ref_s.view(-1)[:256] = torch.arange(256, dtype=torch.uint8)[:ref_s.numel()]
    out = upcast_from_mxfp(ref_v.to(device), ref_s.to(device), dtype, axis)
    ref = upcast_from_mxfp_ref(ref_v, ref_s, dtype, axis)
    a, b = out.cpu().float(), ref.float()
    assert torch.equal(torch.isnan(a), torch.isnan(b))
    assert torch.equal(torch.nan_to_num(a), torch.nan_to_num(b))


def test_all_e2m1_values_roundtrip(device):
    """Every e2m1 value times 2^p, p in [-8, 8), survives quantise -> dequantise (tests/test_mxfp.py:171-205)."""
    grid = torch.tensor([0, 0.5, 1, 1.5, 2, 3, 4, 6])
    grid = torch.cat([grid, -grid])
    rows = []
    for p in range(-8, 8):
        rows.append(torch.cat([grid, grid]) * 2.0**p)
    x = torch.stack(rows)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        xd = x.to(dt).to(device)
        v, s = downcast_to_mxfp(xd, torch.uint8, axis=1)
        back = upcast_from_mxfp(v, s, dt, axis=1)
        assert torch.equal(back, xd)


def test_extreme_values_stay_finite(device):
    x = torch.full((4, 32), 3.3895e38, dtype=torch.bfloat16, device=device)
    v, s = downcast_to_mxfp(x, torch.uint8, axis=1)
    back = upcast_from_mxfp(v, s, torch.bfloat16, axis=1)
    assert torch.isfinite(back).all()
    rv, rs = downcast_to_mxfp_ref(x.cpu(), torch.uint8, 1)
    assert torch.equal(v.cpu(), rv) and torch.equal(s.cpu(), rs)


def test_empty_and_errors(device):
    v, s = downcast_to_mxfp(torch.empty((0, 64), device=device), torch.uint8, axis=1)
    assert v.shape == (0, 32) and s.shape == (0, 2)
    with pytest.raises(AssertionError):
        downcast_to_mxfp(torch.zeros((4, 33), device=device), torch.uint8, axis=1)


def test_pitched_input(device):
    torch.manual_seed(3)
    big = torch.randn(64, 300)
    x = big[:, :256]
    rv, rs = downcast_to_mxfp_ref(x, torch.uint8, 1)
    v, s = downcast_to_mxfp(big.to(device)[:, :256], torch.uint8, axis=1)
    assert torch.equal(v.cpu(), rv) and torch.equal(s.cpu(), rs)


# ---------------------------------------------------------------------------- fp8 values (MXFP8)

FP8_TYPES = [torch.float8_e4m3fn, torch.float8_e5m2]


@pytest.mark.parametrize("shape,axis", [((256, 2880), 1), ((3, 96, 224), -1), ((7, 32), 1), ((2048, 96), 0), ((4, 64, 6), 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("vdt", FP8_TYPES)
@pytest.mark.parametrize("mode", list(DequantScaleRoundingMode))
def test_mxfp8_downcast_matches_oracle(shape, axis, dtype, vdt, mode, device):
    torch.manual_seed(0)
    x = (torch.randn(shape) * torch.exp(torch.randn(shape) * 2)).to(dtype)
    x.view(-1)[::17] = 0
    ref_v, ref_s = downcast_to_mxfp_ref(x, vdt, axis, "up" if mode.value == 0 else "down")
    v, s = downcast_to_mxfp(x.to(device), vdt, axis, DEQUANT_SCALE_ROUNDING_MODE=mode)
    assert v.dtype == vdt and tuple(v.shape) == tuple(x.shape)
    assert torch.equal(s.cpu(), ref_s), "scales differ"
    assert torch.equal(v.cpu().view(torch.uint8), ref_v.contiguous().view(torch.uint8)), "values differ"


@pytest.mark.parametrize("shape,axis", [((128, 512), 1), ((4, 64, 96), 2), ((96, 40), 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("vdt", FP8_TYPES)
def test_mxfp8_upcast_matches_oracle(shape, axis, dtype, vdt, device):
    """Every fp8 byte (NaN codes included) against every scale byte (0 and 0xFF included)."""
    torch.manual_seed(2)
    v = torch.randint(0, 256, shape, dtype=torch.uint8).view(vdt)
    s_shape = list(shape)
    s_shape[axis] //= 32
    s = torch.randint(0, 256, s_shape, dtype=torch.uint8)
    s.view(-1)[:2] = torch.tensor([0, 255], dtype=torch.uint8)
    out = upcast_from_mxfp(v.to(device), s.to(device), dtype, axis)
    ref = upcast_from_mxfp_ref(v, s, dtype, axis)
    a, b = out.cpu().float(), ref.float()
    assert torch.equal(torch.isnan(a), torch.isnan(b))
    assert torch.equal(torch.nan_to_num(a), torch.nan_to_num(b))


@pytest.mark.parametrize("vdt,max_q", [(torch.float8_e4m3fn, 448.0), (torch.float8_e5m2, 57344.0)])
@pytest.mark.parametrize("dst", [torch.float32, torch.bfloat16, torch.float16])
def test_mxfp8_quant_dequant_exact(vdt, max_q, dst, device):
    """The reference's tests/test_mxfp.py:171-205 for the fp8 value types, quantised along a strided axis."""
    top = 128.0 if (vdt == torch.float8_e5m2 and dst == torch.float16) else max_q
    pos = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, top], dtype=dst)
    k = torch.cat([pos, -pos]).reshape(-1, 1)
    w = (k * (2.0**torch.arange(-8, 8, dtype=dst)).reshape(1, -1)).repeat(9, 32)
    w = w.reshape(1, *w.shape).mT.contiguous().mT
    w = torch.nn.functional.pad(w, (0, 0, 0, 16)).to(device)
    q, s = downcast_to_mxfp(w, vdt, axis=1)
    assert torch.equal(upcast_from_mxfp(q, s, dst, axis=1), w)


@pytest.mark.parametrize("anchor", [6.0, 4.0, 1.0, 448.0, 3.0e38])
@pytest.mark.parametrize("axis", [0, 1])
def test_every_bf16_value_against_oracle(anchor, axis, device):
    """All 65536 bfloat16 bit patterns (NaNs and infinities included), 31 to a group next to an anchor that fixes the
    group's scale: codes and scales must equal the oracle's for each of them, along a contiguous and a strided axis."""
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = allv[torch.isfinite(allv.float()) & (allv.float().abs() <= anchor)]
    pad = (-finite.numel()) % 31
    vals = torch.cat([finite, torch.zeros(pad, dtype=torch.bfloat16)]).view(-1, 31)
    x = torch.cat([torch.full((vals.shape[0], 1), anchor, dtype=torch.bfloat16), vals], dim=1)  # [groups, 32]
    if axis == 0:
        x = x.t().contiguous()  # [32, groups]: quantised axis strided
    for vdt in (torch.uint8, torch.float8_e4m3fn, torch.float8_e5m2):
        if vdt != torch.uint8 and axis == 0:
            continue
        rv, rs = downcast_to_mxfp_ref(x, vdt, axis)
        v, s = downcast_to_mxfp(x.to(device), vdt, axis)
        assert torch.equal(s.cpu(), rs)
        assert torch.equal(v.cpu().view(torch.uint8), rv.view(torch.uint8))
