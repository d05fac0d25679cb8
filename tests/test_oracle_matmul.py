"""Pins oracle/matmul_ref.py (grouped matmul, SwiGLU, combine) with checks that a dropped term, a transposed
operand or a wrong index would fail: float64 evaluation with python-level indexing on tiny shapes, one-hot
activations that must reproduce dequantised weight rows bit for bit, zero weights that leave bias*beta*gamma,
and limits of the activation."""
import math

import numpy as np
import pytest
import torch

from oracle import matmul_ref as MR
from oracle import mxfp_ref as MX


def _mx_weights(E, K, N, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(E, K, N, generator=g) * 0.5
    q, s = MX.downcast_to_mxfp_ref(w, torch.uint8, axis=1)
    return q, s, MX.upcast_from_mxfp_ref(q, s, torch.float32, axis=1)


def test_dequantised_weights_are_exact_in_bf16():
    # apply_precision dequantises to bf16 (matmul.py:772-778 of the reference); e2m1 * 2**e needs 2 mantissa bits
    q, s, w32 = _mx_weights(2, 64, 8, 0)
    w16 = MX.upcast_from_mxfp_ref(q, s, torch.bfloat16, axis=1)
    assert torch.equal(w16.float(), w32)


def test_ragged_gather_scatter_against_float64_loops():
    torch.manual_seed(0)
    E, K, N, T, k = 3, 64, 6, 5, 2
    q, s, w = _mx_weights(E, K, N, 1)
    x = torch.randn(T, K).bfloat16()
    bias = torch.randn(E, N)
    sizes = torch.tensor([4, 0, 6], dtype=torch.int32)
    gather = torch.tensor([0, 1, 2, 4, 0, 1, 2, 3, 3, 4], dtype=torch.int32)
    scatter = torch.tensor([3, 7, 1, 9, 0, 2, 4, 5, 6, 8], dtype=torch.int32)
    betas = torch.rand(10)
    gammas = torch.rand(10)
    y = MR.matmul_ref(x, q, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=s,
                      betas=betas, gammas=gammas)
    assert y.dtype == torch.bfloat16 and y.shape == (10, N)
    expert_of_row = [0] * 4 + [2] * 6
    for r in range(10):
        e = expert_of_row[r]
        for n in range(N):
            acc = 0.0
            for kk in range(K):
                acc += float(x[gather[r], kk]) * float(w[e, kk, n])
            want = (acc + float(bias[e, n]) * float(betas[r])) * float(gammas[r])
            got = float(y[scatter[r], n])
            assert abs(got - want) <= 2**-8 * abs(want) + 1e-6, (r, n, got, want)


def test_one_hot_rows_reproduce_weight_rows():
    E, K, N = 2, 96, 10
    q, s, w = _mx_weights(E, K, N, 2)
    x = torch.zeros(6, K, dtype=torch.bfloat16)
    hot = [0, 33, 95, 1, 64, 31]
    for r, kk in enumerate(hot):
        x[r, kk] = 1.0
    y = MR.matmul_ref(x, q, None, slice_sizes=torch.tensor([3, 3], dtype=torch.int32), b_mx_scale=s)
    for r, kk in enumerate(hot):
        assert torch.equal(y[r].float(), w[r // 3, kk])  # a transposed or mis-grouped weight fails here


def test_zero_weights_leave_bias_beta_gamma():
    E, K, N = 2, 32, 4
    q = torch.zeros(E, K // 2, N, dtype=torch.uint8)
    s = torch.full((E, 1, N), 127, dtype=torch.uint8)
    x = torch.randn(5, K).bfloat16()
    bias = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-1.0, -2.0, -3.0, -4.0]])
    betas = torch.tensor([1.0, 0.5, 2.0, 0.0, 1.0])
    gammas = torch.tensor([1.0, 1.0, 0.5, 3.0, -1.0])
    y = MR.matmul_ref(x, q, bias, slice_sizes=torch.tensor([2, 3], dtype=torch.int32), b_mx_scale=s, betas=betas,
                      gammas=gammas)
    e_of = [0, 0, 1, 1, 1]
    want = torch.stack([bias[e_of[r]] * betas[r] * gammas[r] for r in range(5)])
    assert torch.equal(y.float(), want.bfloat16().float())


def test_scatter_minus_one_drops_rows_and_flex_scale():
    torch.manual_seed(3)
    K, N = 32, 4
    w = torch.randn(1, K, N)
    x8 = (torch.randn(4, K)).to(torch.float8_e4m3fn)
    sc = torch.tensor([0.25])
    y = MR.matmul_ref(x8, w, None, slice_sizes=torch.tensor([4], dtype=torch.int32),
                      scatter_indx=torch.tensor([2, -1, 0, 1], dtype=torch.int32), a_flex_scale=sc)
    assert y.dtype == torch.float32  # fp8 + flex scale computes and returns float32 (matmul.py:761-764, 889)
    full = (x8.double() * 0.25) @ w[0].double()
    torch.testing.assert_close(y[2].double(), full[0], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(y[0].double(), full[2], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(y[1].double(), full[3], rtol=1e-5, atol=1e-6)
    assert y[3].eq(0).all()


def test_dense_and_batched_modes():
    torch.manual_seed(4)
    a = torch.randn(3, 7, 16)
    b = torch.randn(3, 16, 5)
    bias = torch.randn(3, 5)
    y = MR.matmul_ref(a, b, bias)
    want = torch.einsum("bmk,bkn->bmn", a.double(), b.double()) + bias[:, None, :].double()
    torch.testing.assert_close(y.double(), want, rtol=1e-5, atol=1e-5)
    y2 = MR.matmul_ref(a[0], b[0], bias[0])
    torch.testing.assert_close(y2, y[0])


def test_swiglu_formula_float64_and_limits():
    torch.manual_seed(5)
    a = torch.randn(9, 16) * 4
    alpha, limit = 1.702, 7.0
    out = MR.swiglu_ref(a, alpha, limit)
    for r in range(9):
        for j in range(8):
            g = min(float(a[r, 2 * j]), limit)          # gate: even column, clamped from above only
            l = max(-limit, min(float(a[r, 2 * j + 1]), limit))
            want = g / (1.0 + math.exp(-alpha * g)) * (l + 1.0)
            assert abs(float(out[r, j]) - want) <= 1e-5 * max(1.0, abs(want))
    far = torch.tensor([[-1e4, 3.0, 50.0, 2.0, 50.0, -50.0]])
    o = MR.swiglu_ref(far, alpha, limit)
    assert o[0, 0].item() == 0.0 or abs(o[0, 0].item()) < 1e-30      # g -> -inf gives 0 (not clamped below)
    assert abs(o[0, 1].item() - 7.0 * (2.0 + 1.0)) < 1e-3             # large g saturates at limit, sigmoid -> 1
    assert abs(o[0, 2].item() - 7.0 * (-7.0 + 1.0)) < 1e-3            # linear clamps on both sides
    nolim = MR.swiglu_ref(far, alpha, None)
    assert abs(nolim[0, 1].item() - 50.0 * 3.0) < 1e-3


def test_fused_swiglu_order():
    # kernel order: activation on the float32 result, then gamma, then the cast
    torch.manual_seed(6)
    K, N = 32, 8
    w = torch.randn(1, K, N)
    x = torch.randn(3, K).bfloat16()
    gam = torch.tensor([0.5, 2.0, -1.0])
    y = MR.matmul_ref(x, w, None, slice_sizes=torch.tensor([3], dtype=torch.int32), gammas=gam,
                      fused_swiglu=(1.702, 7.0))
    z = x.float() @ w[0]
    want = (MR.swiglu_ref(z, 1.702, 7.0) * gam[:, None]).bfloat16()
    assert torch.equal(y, want) and y.shape == (3, N // 2)


def test_reduce_direct_sum():
    torch.manual_seed(7)
    x = torch.randn(6, 4, 10).bfloat16()
    mask = torch.rand(6, 4, 1) > 0.3
    scale = torch.rand(6, 4, 1)
    z = MR.reduce_ref(x, 1, mask=mask, scale=scale)
    for t in range(6):
        for n in range(10):
            acc = np.float32(0)
            for j in range(4):
                if mask[t, j, 0]:
                    acc = np.float32(acc + np.float32(float(x[t, j, n])) * np.float32(float(scale[t, j, 0])))
            assert float(z[t, n]) == float(torch.tensor(float(acc)).bfloat16()), (t, n)
    assert torch.equal(MR.reduce_ref(x, 1), x.float().sum(1).bfloat16())


def test_reduce_mx_small_integers_by_hand():
    """reduce.py:1185-1206: dequantise, sum over `dim`, quantise to MXFP8.  With small integers every step is exact,
    so the result must be the MXFP8 image of the plain integer sum."""
    from oracle.mxfp_ref import downcast_to_mxfp_ref, upcast_from_mxfp_ref
    torch.manual_seed(3)
    x = torch.randint(-6, 7, (5, 3, 64)).float()
    xv, xs = downcast_to_mxfp_ref(x, torch.float8_e4m3fn, axis=-1)
    assert torch.equal(upcast_from_mxfp_ref(xv, xs, torch.float32, axis=-1), x)  # small integers survive MXFP8
    mask = torch.tensor([True, False, True]).reshape(1, 3, 1)
    scale = torch.tensor([2.0, 4.0, 0.5]).reshape(1, 3, 1)
    yv, ys = MR.reduce_mx_ref(xv.contiguous(), xs.contiguous(), 1, mask=mask, scale=scale)
    want = 2.0 * x[:, 0] + 0.5 * x[:, 2]
    wv, ws = downcast_to_mxfp_ref(want, torch.float8_e4m3fn, axis=-1)
    assert torch.equal(ys, ws) and torch.equal(yv.contiguous().view(torch.uint8), wv.contiguous().view(torch.uint8))
    for t in range(5):  # and that image is within half an fp8 step of the exact sum
        got = upcast_from_mxfp_ref(yv, ys, torch.float32, axis=-1)[t]
        assert torch.all((got - want[t]).abs() <= want[t].abs().reshape(2, 32).amax(dim=1).repeat_interleave(32) / 16 + 1e-6)


def test_reduce_general_ref_hand_worked():
    """Two rows, four columns, every optional operand, worked by hand (reduce.py:441-492, flexpoint.py:137-188)."""
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0], [0.5, -1.0, 8.0, 2.0]]])            # [S0=1, R=2, S1=4]
    mask = torch.tensor([[[1, 1, 1, 0], [1, 1, 0, 1]]], dtype=torch.bool)
    scale = torch.tensor([[[2.0], [4.0]]])                                        # per reduced row
    flex = torch.tensor([0.5])
    # terms ((x * flex) * scale), masked: row 0 -> [1, 2, 3, 0], row 1 -> [1, -2, 0, 4]; sums [2, 0, 3, 4]
    y, ymx, actual = MR.reduce_general_ref(x, 1, mask=mask, scale=scale, x_flex_scale=flex)
    assert ymx is None and torch.equal(y, torch.tensor([[2.0, 0.0, 3.0, 4.0]]))
    # plus_a with a = 10 over column pairs: (2 + 10) + (0 + 10) = 22, (3 + 10) + (4 + 10) = 27; global scale 2 -> 44, 54
    y, _, actual = MR.reduce_general_ref(x, 1, mask=mask, scale=scale, x_flex_scale=flex, postprocess=("plus_a", 10.0),
                                         x_global_scale=torch.tensor([2.0]), y_dtype=torch.float8_e4m3fn,
                                         y_expected_scale=torch.tensor([0.125]), y_saturate_inf=True)
    # actual scale is taken before the division: 54 / 448 + 1e-30; 44 / 0.125 = 352, 54 / 0.125 = 432 (both e4m3 numbers... 432
    # lies between 416 and 448 on a grid of 32: ties to even -> 448)
    assert abs(float(actual) - 54.0 / 448.0) < 1e-7
    assert torch.equal(y.float(), torch.tensor([[352.0, 448.0]]))
    # without saturation an overflowing value becomes NaN in float8_e4m3fn, with it the largest finite number
    y_ns, _, _ = MR.reduce_general_ref(x, 1, y_dtype=torch.float8_e4m3fn, y_expected_scale=torch.tensor([0.001]))
    y_s, _, _ = MR.reduce_general_ref(x, 1, y_dtype=torch.float8_e4m3fn, y_expected_scale=torch.tensor([0.001]), y_saturate_inf=True)
    assert torch.isnan(y_ns.float()).all() and torch.equal(y_s.float(), torch.tensor([[448.0, 448.0, 448.0, 448.0]]))


def test_reduce_general_ref_reduces_to_the_pinned_pieces():
    """Without the extra operands it is reduce_ref; with SwiGLU it is swiglu_ref of the float32 sums; the microscaled
    form is reduce_mx_ref; an fp8 input with a flex scale is the scaled sum of its exact float32 values."""
    from oracle.mxfp_ref import downcast_to_mxfp_ref
    torch.manual_seed(0)
    x = torch.randn(5, 3, 64)
    mask = torch.rand(5, 3, 1) > 0.3
    scale = torch.rand(1, 3, 1) + 0.5
    y, _, _ = MR.reduce_general_ref(x, 1, mask=mask, scale=scale)
    assert torch.equal(y, MR.reduce_ref(x, 1, mask=mask, scale=scale))
    y, _, _ = MR.reduce_general_ref(x, 1, postprocess=("swiglu", 1.702, 7.0))
    assert torch.equal(y, MR.swiglu_ref(MR.reduce_ref(x, 1), 1.702, 7.0))
    xv, xs = downcast_to_mxfp_ref(x, torch.float8_e4m3fn, axis=-1)
    v, s2, _ = MR.reduce_general_ref(xv.contiguous(), 0, mask=mask, x_mxscale=xs.contiguous(), y_has_mx=True)
    rv, rs = MR.reduce_mx_ref(xv.contiguous(), xs.contiguous(), 0, mask=mask)
    assert torch.equal(v.view(torch.uint8), rv.view(torch.uint8)) and torch.equal(s2, rs)
    x8 = (x / 2).to(torch.float8_e5m2)
    y, _, actual = MR.reduce_general_ref(x8, 1, x_flex_scale=torch.tensor([2.0]), y_dtype=torch.float32)
    want = (x8.float() * 2.0)[:, 0] + (x8.float() * 2.0)[:, 1] + (x8.float() * 2.0)[:, 2]
    assert torch.equal(y, want)
    assert abs(float(actual) - (float(want.abs().max()) / 3.4028234663852886e38 + 1e-30)) < 1e-36


def test_reduce_general_ref_sign_of_zero_and_unpadded_rows():
    """What IEEE arithmetic makes of the reference kernel's start of the sum (reduce.py:137, 423-424, 466-470), worked by
    hand: up to 8 entries the first term is the initial value, so -0.0 survives; a longer axis starts from +0.0 and
    -0.0 + ... + -0.0 added to +0.0 is +0.0; a scale goes through fma(x, s, +0.0), and (-0.0 * s) + 0.0 is +0.0; a
    masked first entry is loaded as +0.0, and +0.0 + -0.0 is +0.0."""
    neg = lambda t: torch.signbit(t).tolist()
    one = torch.full((1, 1, 2), -0.0)
    y, _, _ = MR.reduce_general_ref(one, 1)
    assert neg(y) == [[True, True]]
    four = torch.full((1, 4, 2), -0.0)
    y, _, _ = MR.reduce_general_ref(four, 1)
    assert neg(y) == [[True, True]]
    nine = torch.full((1, 9, 2), -0.0)
    y, _, _ = MR.reduce_general_ref(nine, 1)
    assert neg(y) == [[False, False]]
    y, _, _ = MR.reduce_general_ref(four, 1, scale=torch.ones(1, 4, 1))
    assert neg(y) == [[False, False]]
    mask = torch.tensor([[[0, 1], [1, 1], [1, 1], [1, 1]]], dtype=torch.bool)
    y, _, _ = MR.reduce_general_ref(four, 1, mask=mask)
    assert neg(y) == [[False, True]]
    # only the first `unpadded_batch_size` entries of the first kept axis are reduced (tests/test_reduce.py:156-176 of the
    # reference: y_ref = x[:, :unpadded, :].sum(0))
    x = torch.arange(2 * 5 * 3, dtype=torch.float32).reshape(2, 5, 3)
    y, _, _ = MR.reduce_general_ref(x, 0, unpadded_batch_size=torch.tensor(3))
    assert torch.equal(y, x[0, :3] + x[1, :3])
