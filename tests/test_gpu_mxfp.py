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
    """Every finite bfloat16 bit pattern up to the anchor, 31 to a group next to an anchor that fixes the group's
    scale: codes and scales must equal the oracle's for each of them, along a contiguous and a strided axis.
    (Non-finite inputs are outside the contract: the reference's own twins disagree on them.)"""
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


# ---------------------------------------------------------------------------- the e2m1 rounding of float32 / float16 sources
# The kernels round with the hardware conversion (v_cvt_scalef32_pk_fp4_f32); the reference's bit path (restated in
# oracle/mxfp_ref.py:e2m1_codes_from_f32 and pinned on the CPU by an exact-rational brute force) is round to nearest,
# ties to even.  The cases below are the ones where the two could part: values one ulp either side of every
# midpoint of the e2m1 grid, at every scale a float32 group can have, tiny and subnormal inputs, signed zeros.

E2M1_MIDPOINTS = (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)


def _check_against_oracle(x, axis, device, vdt=torch.uint8):
    rv, rs = downcast_to_mxfp_ref(x, vdt, axis)
    v, s = downcast_to_mxfp(x.to(device), vdt, axis)
    assert torch.equal(s.cpu(), rs), "scales differ"
    bad = (v.cpu().view(torch.uint8) != rv.contiguous().view(torch.uint8)).nonzero()
    assert bad.numel() == 0, f"{bad.shape[0]} bytes differ, first at {bad[0].tolist()}"


@pytest.mark.parametrize("axis", [0, 1])
def test_f32_tie_neighbours_at_every_scale(axis, device):
    """Anchor 6 * 2^e fixes the scale 2^e of a group; its other members are (midpoint -1 ulp, midpoint, midpoint +1 ulp)
    * 2^e of either sign for all seven midpoints, for every e at which they are normal float32 numbers."""
    mids = torch.tensor(E2M1_MIDPOINTS, dtype=torch.float32)
    bits = mids.view(torch.int32)
    cand = torch.stack([(bits - 1).view(torch.float32), mids, (bits + 1).view(torch.float32)], dim=1).reshape(-1)  # 21
    cand = torch.cat([cand, -cand])  # 42 values, exact multiples of 2^-25
    groups = []
    for e in range(-122, 125):
        sc = torch.tensor(2.0, dtype=torch.float64)**e
        vals = (cand.double() * sc).float()
        assert torch.equal(vals.double(), cand.double() * sc)  # scaling by a power of two is exact here
        for part in (vals[:21], vals[21:]):
            g = torch.zeros(32, dtype=torch.float32)
            g[0] = float(6.0 * sc)
            g[1:22] = part
            groups.append(g)
    x = torch.stack(groups)  # [groups, 32]
    if axis == 0:
        x = x.t().contiguous()
    _check_against_oracle(x, axis, device)


@pytest.mark.parametrize("axis", [0, 1])
def test_f32_tiny_subnormal_and_signed_zero_inputs(axis, device):
    """Members far below the group's scale round to a zero that keeps its sign (the reference's bit path carries the
    sign bit through); subnormal inputs and whole groups of subnormals (scale byte 0 or 1) included."""
    tiny = torch.tensor([0.0, -0.0, 1e-45, -1e-45, 1e-40, -1e-40, 1.17549435e-38, -1.17549435e-38, 1e-30, -1e-30, 0.24999999, -0.24999999,
                         0.25, -0.25, 0.25000003, -0.25000003], dtype=torch.float32)
    groups = []
    for anchor in (1.0, 6.0, 5.9999995, 1e-30, 1.17549435e-38, 3e-39, 1e-44, 0.0, 3.0e38):
        g = torch.zeros(32, dtype=torch.float32)
        g[0] = anchor
        g[1:17] = tiny if anchor >= 1e-30 else tiny * 0 + torch.tensor([0.0, -0.0, 1e-45, -1e-45] * 4, dtype=torch.float32)
        g[17:] = torch.tensor([anchor * f for f in (-1.0, 0.5, -0.5, 0.75, -0.75, 0.3, -0.3, 0.2, -0.2, 0.1, -0.1, 0.04, -0.04, 0.9, -0.9)],
                              dtype=torch.float32)
        groups.append(g)
    x = torch.stack(groups)
    if axis == 0:
        x = x.t().contiguous()
    _check_against_oracle(x, axis, device)


def test_f32_random_bit_patterns(device):
    """2^24 random finite float32 bit patterns (every exponent, so most members vanish against their group's maximum)
    and 2^22 values whose exponents stay within six binades of their group's anchor (so most members land on the
    grid proper), against the oracle."""
    g = torch.Generator().manual_seed(7)
    bits = torch.randint(-2**31, 2**31, (2**24, ), generator=g, dtype=torch.int64).to(torch.int32)
    x = bits.view(torch.float32)
    x = torch.where(torch.isfinite(x), x, torch.zeros_like(x)).view(-1, 4096)
    _check_against_oracle(x, 1, device)
    n = 2**22
    mant = torch.randint(0, 2**23, (n, ), generator=g, dtype=torch.int64)
    sign = torch.randint(0, 2, (n, ), generator=g, dtype=torch.int64) << 31
    base = torch.randint(8, 250, (n // 32, 1), generator=g, dtype=torch.int64)
    expo = (base - torch.randint(0, 7, (n // 32, 32), generator=g, dtype=torch.int64)).reshape(-1)
    y = (sign | (expo << 23) | mant).to(torch.int32).view(torch.float32).view(-1, 2048)
    _check_against_oracle(y, 1, device)
    _check_against_oracle(y[:4096].t().contiguous(), 0, device)  # the same values along a strided axis


@pytest.mark.parametrize("anchor", [6.0, 4.0, 1.0, 448.0, 65504.0, 6.1e-5, 6e-8])
@pytest.mark.parametrize("axis", [0, 1])
def test_every_f16_value_against_oracle(anchor, axis, device):
    """Every finite float16 bit pattern (subnormals included) up to the anchor, as in the bfloat16 test above."""
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    finite = allv[torch.isfinite(allv.float()) & (allv.float().abs() <= anchor)]
    pad = (-finite.numel()) % 31
    vals = torch.cat([finite, torch.zeros(pad, dtype=torch.float16)]).view(-1, 31)
    x = torch.cat([torch.full((vals.shape[0], 1), anchor, dtype=torch.float16), vals], dim=1)
    if axis == 0:
        x = x.t().contiguous()
    for vdt in (torch.uint8, torch.float8_e4m3fn, torch.float8_e5m2):
        if vdt != torch.uint8 and axis == 0:
            continue
        _check_against_oracle(x, axis, device, vdt)
