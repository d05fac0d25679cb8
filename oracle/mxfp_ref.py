"""CPU oracle: MXFP quantise / dequantise.  Test infrastructure, never shipped.

Restates numerics_details/mxfp.py:212-363 (downcast_to_mxfp_torch) and
:366-449 (cvt_e2m1_to_fp32, upcast_from_mxfp_torch) of the reference with numpy
integer arithmetic.  Inputs and outputs are torch CPU tensors so bf16 / fp8
dtypes travel unchanged.
"""
import numpy as np
import torch

MXFP_BLOCK = 32
E2M1_GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)  # mxfp.py:373
_MAX_Q = {"e2m1": 6.0, "e4m3": 448.0, "e5m2": 57344.0}  # mxfp.py:206-209
_MAX_Q_POW2 = {"e2m1": 4.0, "e4m3": 256.0, "e5m2": 32768.0}  # _downcast_to_mxfp.py:24-31


def _kind(out_dtype):
    if out_dtype in (torch.uint8, "e2m1"):
        return "e2m1"
    if out_dtype in (torch.float8_e4m3fn, "e4m3"):
        return "e4m3"
    if out_dtype in (torch.float8_e5m2, "e5m2"):
        return "e5m2"
    raise ValueError(f"unsupported mx value type {out_dtype}")


def e2m1_codes_from_f32(q: np.ndarray) -> np.ndarray:
    """fp32 -> 4-bit e2m1 code (sign in bit 3), round-to-nearest-even, saturating.

    Follows the bit path of mxfp.py:319-347: the fp32 exponent is re-biased from
    127 to 1, values below 1.0 become e2m1 subnormals by shifting the mantissa
    (with the implicit one made explicit), the two mantissa bits kept are
    `m2bits`, bit 0 of them is the guard bit, everything shifted out is sticky.
    A shift of 32 or more yields 0, which is what torch's `>>` on int32 gives.
    """
    u = np.ascontiguousarray(q, dtype=np.float32).view(np.uint32).astype(np.int64)
    sign = (u >> 31) & 1
    exp = (u >> 23) & 0xFF
    man = u & 0x7FFFFF
    below_one = exp < 127
    shift = 127 - exp - 1  # >= 0 where below_one
    man_sub_full = 0x400000 | (man >> 1)
    sh = np.clip(shift, 0, 63)
    man_sub = np.where(sh >= 32, 0, man_sub_full >> np.minimum(sh, 31))
    lost_sub = ((man & 1) != 0) | ((man_sub_full & ((np.int64(1) << np.minimum(sh, 31)) - 1)) != 0)
    mant = np.where(below_one, man_sub, man)
    sticky = (below_one & lost_sub) | ((mant & 0x1FFFFF) != 0)
    e = np.maximum(exp, 126) - 126
    m2 = (mant >> 21) & 3
    guard = m2 & 1
    keep_lsb = (m2 >> 1) & 1
    inc = guard & (sticky.astype(np.int64) | keep_lsb)
    mag = np.minimum((((e << 2) | m2) + inc) >> 1, 7)
    return ((sign << 3) | mag).astype(np.uint8)


def downcast_to_mxfp_ref(x: torch.Tensor, out_dtype, axis: int, rounding: str = "up"):
    """Returns (values, scales) like downcast_to_mxfp_torch (mxfp.py:212-363).

    values: uint8 with two e2m1 codes per byte (even index in the low nibble,
    mxfp.py:350-353) or an fp8 tensor; scales: uint8 e8m0, one per 32 elements
    along `axis`.  `rounding` is "up" (ROUND_UP, :283-291) or "down".
    Both outputs are returned with `axis` in its original position.
    """
    kind = _kind(out_dtype)
    ndim = x.ndim
    axis = axis % ndim
    assert x.dtype in (torch.float32, torch.bfloat16, torch.float16)
    src = x.transpose(axis, ndim - 1).to(torch.float32).contiguous().numpy()
    L = src.shape[-1]
    if kind == "e2m1":
        assert L % 2 == 0
    G = -(-L // MXFP_BLOCK)
    pad = G * MXFP_BLOCK - L
    data = np.pad(src, [(0, 0)] * (ndim - 1) + [(0, pad)])
    mag = np.abs(data)
    if pad:
        mag[..., L:] = -1.0  # padding never wins the max (mxfp.py:273-274)
    groups = data.reshape(*data.shape[:-1], G, MXFP_BLOCK)
    gmax = mag.reshape(groups.shape).max(axis=-1, keepdims=True).astype(np.float32)
    if rounding == "up":
        ds = (gmax / np.float32(_MAX_Q[kind])).astype(np.float32)
        sbits = (ds.view(np.uint32) + np.uint32(0x007FFFFF)) & np.uint32(0x7F800000)
    else:
        ds = (gmax / np.float32(_MAX_Q_POW2[kind])).astype(np.float32)
        sbits = ds.view(np.uint32) & np.uint32(0x7F800000)
    ds_r = sbits.view(np.float32)
    with np.errstate(divide="ignore"):
        qs = np.where(ds_r == 0, np.float32(0), np.float32(1) / ds_r).astype(np.float32)
    q = (groups * qs).astype(np.float32).reshape(data.shape)[..., :L]
    scales = (sbits >> np.uint32(23)).astype(np.uint8).reshape(*data.shape[:-1], G)
    if kind == "e2m1":
        codes = e2m1_codes_from_f32(q)
        vals = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
        vals_t = torch.from_numpy(vals)
    else:
        mq = _MAX_Q[kind]
        tdt = torch.float8_e4m3fn if kind == "e4m3" else torch.float8_e5m2
        vals_t = torch.from_numpy(np.clip(q, -mq, mq)).to(tdt)  # mxfp.py:313-316
    scales_t = torch.from_numpy(scales)
    return vals_t.transpose(axis, ndim - 1), scales_t.transpose(axis, ndim - 1)


def e2m1_unpack_f32(packed: np.ndarray) -> np.ndarray:
    """uint8 [..., n] -> float32 [..., 2n]; mxfp.py:366-381."""
    table = np.array(E2M1_GRID + tuple(-v for v in E2M1_GRID), dtype=np.float32)
    lo = table[packed & 0xF]
    hi = table[(packed >> 4) & 0xF]
    return np.stack([lo, hi], axis=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def upcast_from_mxfp_ref(values: torch.Tensor, scales: torch.Tensor, target_dtype, axis: int,
                         nan_on_ff: bool = True):
    """Dequantise (values, e8m0 scales) along `axis` to `target_dtype`.

    Follows mxfp.py:384-449: value * float32_from_bits(scale << 23), clamped to
    the finite range of the target, then cast.  A scale byte of 0 therefore
    multiplies by +0.0 (not 2^-127).  With `nan_on_ff` the OCP NaN scale 0xFF
    yields NaN for the whole group, which is what the reference's GPU kernel
    does (mxfp_details/_upcast_from_mxfp.py:166-168); its torch twin instead
    lets 0xFF act as +inf (so x*inf clamps to the largest finite value).  The
    reference's tests never feed 0xFF; this oracle pins the GPU behaviour and
    keeps the twin's available through nan_on_ff=False.
    """
    ndim = values.ndim
    axis = axis % ndim
    assert scales.dtype == torch.uint8
    v = values.transpose(axis, ndim - 1).contiguous()
    s = scales.transpose(axis, ndim - 1).contiguous().numpy()
    if values.dtype == torch.uint8:
        f = e2m1_unpack_f32(v.numpy())
    else:
        f = v.to(torch.float32).numpy()
    L = f.shape[-1]
    if L == 0:
        return torch.from_numpy(f).to(target_dtype).transpose(axis, ndim - 1).contiguous()
    G = -(-L // MXFP_BLOCK)
    assert s.shape[-1] == G, (s.shape, G)
    pad = G * MXFP_BLOCK - L
    fp = np.pad(f, [(0, 0)] * (ndim - 1) + [(0, pad)]).reshape(*f.shape[:-1], G, MXFP_BLOCK)
    mult = (s.astype(np.uint32) << np.uint32(23)).view(np.float32)[..., None]
    fin = torch.finfo(target_dtype)
    with np.errstate(invalid="ignore", over="ignore"):
        out = np.clip(fp * mult, np.float32(fin.min), np.float32(fin.max)).astype(np.float32)
    if values.dtype == torch.float8_e5m2:
        out = np.where(np.isinf(fp), fp, out)  # mxfp.py:438-440
    if nan_on_ff:
        out = np.where((s == 0xFF)[..., None], np.float32(np.nan), out)
    out = out.reshape(*f.shape[:-1], G * MXFP_BLOCK)[..., :L]
    return torch.from_numpy(np.ascontiguousarray(out)).to(target_dtype).transpose(axis, ndim - 1)
