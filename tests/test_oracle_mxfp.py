"""Pins oracle/mxfp_ref.py against evidence that does not come from the oracle itself:
the literals held by the reference's tests (tests/test_mxfp.py:92-205 of the reference's triton_kernels
package), the e2m1 value table (numerics_details/mxfp.py:373), closed forms of the e8m0 scale, and a
brute-force nearest-even rounding over every bf16 value written with exact rational arithmetic."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import mxfp_ref as MX

GRID = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def _roundtrip(x, dt, rounding="up", axis=1):
    q, s = MX.downcast_to_mxfp_ref(x, torch.uint8, axis=axis, rounding=rounding)
    return q, s, MX.upcast_from_mxfp_ref(q, s, dt, axis=axis)


@pytest.mark.parametrize("dt,ulp_case", [(torch.bfloat16, 0.251953125), (torch.float16, 0.250244140625),
                                         (torch.float32, 0.2500000298023223877)])
def test_reference_rounding_literals(dt, ulp_case):
    # tests/test_mxfp.py:100-114 of the reference: group max 6 -> scale 1; ties go to the even code.
    x = torch.tensor([6, 0, 0.24, 0.25, 0.75, 0.99, 1.2, 1.3, -1.25, ulp_case] + [0] * 22, dtype=dt).view(1, -1, 1)
    q, s, d = _roundtrip(x, dt)
    assert s.flatten().tolist() == [127]
    assert d.flatten().tolist() == [6, 0, 0, 0.0, 1.0, 1.0, 1.0, 1.5, -1.0, 0.5] + [0] * 22
    # packing: even index in the low nibble (mxfp.py:350-353).  codes: 6->7, 0->0, .24->0, .25->0, 1.0->2 ...
    assert q.flatten().tolist()[:5] == [0x07, 0x00, 0x22, 0x32, 0x1A]


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_reference_round_down_literal(dt):
    # tests/test_mxfp.py:128-141: max 33 with ROUND_DOWN -> scale 2**3, byte 130, the rest reconstructs exactly.
    x = torch.tensor([33.0, 24.0, 16.0, 8.0, 4.0, 0.0, -32.0, 0.0] + [0] * 24).bfloat16().view(1, -1, 1)
    q, s, d = _roundtrip(x, dt, rounding="down")
    assert s.item() == 130
    assert torch.equal(d[0, 1:, :].float(), x[0, 1:, :].float())
    assert d[0, 0, 0].item() == 32.0  # 33/8 = 4.125 rounds to 4


def test_reference_worked_scale_example():
    # numerics_details/mxfp.py:430-435 works a scale byte of 247 (2**120) through the upcast.
    q = torch.tensor([[0x72] + [0] * 15], dtype=torch.uint8)  # codes 2 (1.0) and 7 (6.0)
    s = torch.tensor([[247]], dtype=torch.uint8)
    d = MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=1)
    assert d[0, 0].item() == 2.0**120 and d[0, 1].item() == 6 * 2.0**120


@pytest.mark.parametrize("dt,big", [(torch.float16, 65470.0), (torch.bfloat16, 3.3895e38), (torch.float32, 3.3895e38)])
def test_reference_extreme_values_stay_finite(dt, big):
    # tests/test_mxfp.py:154-168
    x = torch.tensor([big, big] + [0] * 30, dtype=dt)
    q, s = MX.downcast_to_mxfp_ref(x, torch.uint8, axis=-1)
    d = MX.upcast_from_mxfp_ref(q, s, dt, axis=-1)
    assert not d.isinf().any() and not d.isnan().any()
    assert d[0].item() == torch.finfo(dt).max or d[0].float().item() >= 0.5 * big


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_reference_exact_roundtrip_of_grid_times_pow2(dt):
    # tests/test_mxfp.py:171-205: every e2m1 value times 2**p, p in [-8, 8), survives quantise -> dequantise.
    vals = torch.tensor(GRID + [-v for v in GRID])
    rows = []
    for p in range(-8, 8):
        rows.append(torch.cat([vals * 2.0**p, vals.flip(0) * 2.0**p]))  # 32 per group, max is 6*2**p
    x = torch.stack(rows).to(dt)
    q, s, d = _roundtrip(x, dt)
    assert torch.equal(d, x)
    assert s.flatten().tolist() == [127 + p for p in range(-8, 8)]


def test_value_table():
    packed = np.arange(256, dtype=np.uint8)[None]
    f = MX.e2m1_unpack_f32(packed)[0]
    for b in range(256):
        for half, code in enumerate((b & 0xF, b >> 4)):
            want = GRID[code & 7] * (-1 if code & 8 else 1)
            got = f[2 * b + half]
            assert got == want and (np.signbit(got) == bool(code & 8))


def _rtne_code_exact(v: float) -> int:
    """Nearest e2m1 magnitude with ties to the even code, saturating, in exact rationals."""
    a = Fraction(abs(v))
    best, best_d = None, None
    for code, g in enumerate(GRID):
        d = abs(a - Fraction(g))
        if best is None or d < best_d or (d == best_d and code % 2 == 0 and best % 2 == 1):
            best, best_d = code, d
    if a >= 6:
        best = 7
    return best | (8 if np.signbit(np.float32(v)) else 0)


def test_e2m1_rounding_brute_force_all_bf16():
    bits = np.arange(65536, dtype=np.uint32) << 16
    f = bits.view(np.float32)
    finite = np.isfinite(f)
    got = MX.e2m1_codes_from_f32(f[finite])
    want = np.array([_rtne_code_exact(float(v)) for v in f[finite]], dtype=np.uint8)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (f[finite][bad[:5]], got[bad[:5]], want[bad[:5]])


def test_e2m1_rounding_fp32_neighbours_of_every_tie():
    # the seven midpoints and their fp32 neighbours: the guard/sticky logic must split exactly there.
    mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    xs = []
    for m in mids:
        m32 = np.float32(m)
        xs += [np.nextafter(m32, np.float32(0)), m32, np.nextafter(m32, np.float32(10))]
    xs = np.array(xs + [-x for x in xs], dtype=np.float32)
    got = MX.e2m1_codes_from_f32(xs)
    want = np.array([_rtne_code_exact(float(v)) for v in xs], dtype=np.uint8)
    assert np.array_equal(got, want)


def _scale_closed_form(m: float, rounding: str) -> int:
    """ROUND_UP: smallest power of two 2**e with m <= 6*2**e; ROUND_DOWN: largest with 4*2**e <= m."""
    if m == 0:
        return 0
    fm = Fraction(m)
    e = -140
    if rounding == "up":
        while Fraction(6) * Fraction(2)**e < fm:
            e += 1
    else:
        while Fraction(4) * Fraction(2)**(e + 1) <= fm:
            e += 1
    return max(e + 127, 0)


@pytest.mark.parametrize("rounding", ["up", "down"])
def test_scale_byte_closed_form(rounding):
    rng = np.random.default_rng(0)
    bits = rng.integers(0x0400, 0x7F00, size=400).astype(np.uint32) << 16  # positive normal bf16 values
    ms = np.concatenate([bits.view(np.float32), np.float32([6, 12, 3, 4, 8, 1.5, 0.75, 6 * 2.0**-10, 4 * 2.0**20, 0])])
    for m in ms:
        x = torch.zeros(1, 32)
        x[0, 7] = float(m)
        _, s = MX.downcast_to_mxfp_ref(x, torch.uint8, axis=1, rounding=rounding)
        # fp32 division m/6 is correctly rounded; an exact power of two can only arise from an exact quotient
        # for ROUND_UP (6 is not a power of two), so the closed form holds for every input except when the
        # rounded quotient crosses a binade: allow that single case explicitly.
        want = _scale_closed_form(float(m), rounding)
        got = int(s.item())
        if rounding == "up" and got != want:
            q = np.float32(m) / np.float32(6)
            assert q.view(np.uint32) & 0x7FFFFF == 0 and got == want - 1, (m, got, want)
        else:
            assert got == want, (m, got, want)


def test_zero_group_and_scale_zero():
    x = torch.zeros(2, 64)
    x[1, 3] = 1.0
    q, s = MX.downcast_to_mxfp_ref(x, torch.uint8, axis=1)
    assert s.tolist() == [[0, 0], [125, 0]]  # 1/6 -> 2**-2
    assert q[0].eq(0).all()
    d = MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=1)
    assert d[1, 3].item() == 1.0 and d.sum().item() == 1.0
    # a scale byte of zero multiplies by +0.0 (bit pattern 0 << 23), not by 2**-127
    q2 = torch.full((1, 16), 0x77, dtype=torch.uint8)
    d2 = MX.upcast_from_mxfp_ref(q2, torch.zeros(1, 1, dtype=torch.uint8), torch.float32, axis=1)
    assert d2.eq(0).all()


def test_scale_ff_behaviours():
    q = torch.tensor([[0x20] + [0] * 15], dtype=torch.uint8)
    s = torch.tensor([[255]], dtype=torch.uint8)
    assert MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=1).isnan().all()
    twin = MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=1, nan_on_ff=False)
    assert twin[0, 1].item() == torch.finfo(torch.float32).max and twin[0, 0].isnan()


@pytest.mark.parametrize("shape,axis", [((3, 64, 5), 1), ((64, 7), 0), ((2, 3, 96), -1), ((1, 32, 1), 1)])
def test_layout_and_axis(shape, axis):
    torch.manual_seed(0)
    x = torch.randn(shape)
    q, s = MX.downcast_to_mxfp_ref(x, torch.uint8, axis=axis)
    ax = axis % len(shape)
    want_q = list(shape)
    want_q[ax] //= 2
    want_s = list(shape)
    want_s[ax] //= 32
    assert list(q.shape) == want_q and list(s.shape) == want_s
    # quantising along `axis` equals quantising the transposed tensor along its last axis
    q2, s2 = MX.downcast_to_mxfp_ref(x.transpose(ax, -1).contiguous(), torch.uint8, axis=-1)
    assert torch.equal(q, q2.transpose(ax, -1)) and torch.equal(s, s2.transpose(ax, -1))
    # dequantised error bound: half a grid step (at most 1.0 in scaled units) times the scale
    d = MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=axis)
    sc = torch.from_numpy((s.contiguous().numpy().astype(np.uint32) << 23).view(np.float32)).repeat_interleave(32, dim=ax)
    assert ((d - x).abs() <= sc * 1.0 + 1e-30).all()


def test_ragged_tail_group():
    # a last group shorter than 32 is padded; the padding never wins the max (mxfp.py:273-274)
    x = torch.zeros(1, 40)
    x[0, 35] = 3.0
    q, s = MX.downcast_to_mxfp_ref(x, torch.uint8, axis=1)
    assert list(q.shape) == [1, 20] and s.tolist() == [[0, 126]]
    d = MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=1)
    assert d[0, 35].item() == 3.0


# ---------------------------------------------------------------------------- fp8 values (MXFP8)

FP8_KINDS = [(torch.float8_e4m3fn, 448.0), (torch.float8_e5m2, 57344.0)]


@pytest.mark.parametrize("vdt,max_q", FP8_KINDS)
@pytest.mark.parametrize("dst", [torch.float32, torch.bfloat16, torch.float16])
def test_fp8_representable_values_roundtrip(vdt, max_q, dst):
    """tests/test_mxfp.py:171-205 of the reference for the fp8 value types: {0, .5, 1, 1.5, 2, 3, 4, max} x 2^[-8, 8)
    survive quantise -> dequantise exactly (fp16 cannot hold the e5m2 range: max 128 there, as in the reference)."""
    top = 128.0 if (vdt == torch.float8_e5m2 and dst == torch.float16) else max_q
    pos = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, top], dtype=dst)
    k = torch.cat([pos, -pos]).reshape(-1, 1)
    w = (k * (2.0**torch.arange(-8, 8, dtype=dst)).reshape(1, -1)).repeat(9, 32)
    w = torch.nn.functional.pad(w.reshape(1, *w.shape), (0, 0, 0, 16))
    v, s = MX.downcast_to_mxfp_ref(w, vdt, axis=1)
    assert v.dtype == vdt and s.dtype == torch.uint8 and tuple(s.shape) == (1, w.shape[1] // 32, w.shape[2])
    assert torch.equal(MX.upcast_from_mxfp_ref(v, s, dst, axis=1), w)


@pytest.mark.parametrize("vdt,max_q", FP8_KINDS)
@pytest.mark.parametrize("dst,big", [(torch.float16, 65470.0), (torch.bfloat16, 3.3895e38), (torch.float32, 3.3895e38)])
def test_fp8_extreme_values_stay_finite(vdt, max_q, dst, big):
    """tests/test_mxfp.py:154-168."""
    x = torch.tensor([big, big] + [0.0] * 30, dtype=dst)
    v, s = MX.downcast_to_mxfp_ref(x, vdt, axis=-1)
    out = MX.upcast_from_mxfp_ref(v, s, dst, axis=-1)
    assert not out.isinf().any() and not out.isnan().any()


@pytest.mark.parametrize("vdt,max_q", FP8_KINDS)
def test_fp8_scale_closed_form_and_nearest_value(vdt, max_q):
    """ROUND_UP scale = smallest power of two with max / scale <= max_q; every value is the fp8 number nearest to
    x / scale (ties to the even code), found by brute force over all 256 codes decoded by torch."""
    torch.manual_seed(0)
    x = torch.randn(64, 32) * torch.exp(torch.randn(64, 1) * 3)
    v, s = MX.downcast_to_mxfp_ref(x, vdt, axis=1)
    table = torch.arange(256, dtype=torch.uint8).view(vdt).float()
    finite = torch.isfinite(table)
    for r in range(64):
        m = float(x[r].abs().max())
        e = int(s[r, 0]) - 127
        assert m / 2.0**e <= max_q and (m / 2.0**(e - 1) > max_q)
        q = (x[r].double() / 2.0**e)
        d = (table[finite].double()[None, :] - q[:, None]).abs()
        best = d.min(dim=1).values
        got = v[r].float().double()
        assert torch.all((got - q).abs() <= best + 1e-300)
        # ties: the chosen code has an even mantissa bit pattern
        tie = (d <= best[:, None]).sum(dim=1) > 1
        if tie.any():
            assert torch.all((v[r].view(torch.uint8)[tie] & 1) == 0)


def test_fp8_round_down_uses_largest_power_of_two():
    """mxfp_details/_downcast_to_mxfp.py:24-31: ROUND_DOWN divides by 256 (e4m3) / 32768 (e5m2) and truncates."""
    x = torch.zeros(1, 32)
    x[0, 0] = 300.0
    for vdt, p2 in ((torch.float8_e4m3fn, 256.0), (torch.float8_e5m2, 32768.0)):
        _, s = MX.downcast_to_mxfp_ref(x, vdt, axis=1, rounding="down")
        import math
        assert int(s[0, 0]) == 127 + math.floor(math.log2(300.0 / p2))
