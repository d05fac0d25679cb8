"""GPU parity: matmul (bf16/fp16 x MXFP4, dense and ragged, gather/scatter, bias/beta/gamma, fused SwiGLU)
through the C ABI vs the CPU oracle.  Tolerance: rtol 1e-2 / atol 1e-2 (bf16 out, fp32 accumulate), plus the
reference's own measure (max relative error 3e-2 for mxfp4 weights, tests/test_matmul.py:625-626)."""
import pytest
import torch

from oracle import matmul_ref as MR
from oracle import routing_ref as RR
from oracle.mxfp_ref import downcast_to_mxfp_ref
from triton_amd.matmul import FlexCtx, FnSpecs, FusedActivation, InFlexData, PrecisionConfig, matmul, matmul_ogs
from triton_amd.matmul_details.opt_flags import scoped_opt_flags_constraints
from triton_amd.numerics_details.mxfp import downcast_to_mxfp
from triton_amd.routing import routing
from triton_amd.swiglu import swiglu_fn
from triton_amd.tensor import FP4, convert_layout, make_ragged_tensor_metadata, wrap_torch_tensor
from triton_amd.tensor_details.layout import CDNA4MXValueLayout
from triton_amd.testing import assert_close

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2


def quantize_w(w_cpu, device):
    """fp32 [E, K, N] -> MXFP4 along K on the GPU; checks the codes against the oracle on the way."""
    v, s = downcast_to_mxfp(w_cpu.to(device), torch.uint8, axis=-2)
    rv, rs = downcast_to_mxfp_ref(w_cpu, torch.uint8, axis=-2)
    assert torch.equal(v.cpu(), rv) and torch.equal(s.cpu(), rs)
    return v, s, rv, rs


def check(out, ref):
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL)
    assert_close(ref, out.cpu(), maxtol=3e-2, verbose=False)


def swiglu_act(alpha, limit):
    return FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (alpha, limit))


def test_alias():
    assert matmul_ogs is matmul


@pytest.mark.parametrize("M,K,N", [(256, 2048, 4096), (16, 64, 64), (33, 96, 200), (130, 192, 520), (1, 32, 16),
                                   (15, 96, 66), (40, 160, 322)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dense(M, K, N, dtype, device):
    """(256, 2048, 4096) is BASELINE config 1; (15, 96, 66) and (40, 160, 322) have scale images whose size is not a
    multiple of four bytes (the last columns' scales sit in a partial dword)."""
    torch.manual_seed(0)
    x = torch.randn(M, K).to(dtype)
    w = torch.randn(K, N) * 0.02
    bias = (torch.randn(N) * 0.01).to(torch.bfloat16)
    v, s, rv, rs = quantize_w(w, device)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    out = matmul(x.to(device), v, bias.to(device), precision_config=pc)
    ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs)
    assert out.dtype == dtype and tuple(out.shape) == (M, N)
    check(out, ref)


def test_dense_exact_special_cases(device):
    """One-hot rows pick dequantised weight rows exactly; zero weights give bias*beta*gamma."""
    torch.manual_seed(1)
    K, N = 128, 256
    w = torch.randn(K, N)
    v, s, rv, rs = quantize_w(w, device)
    x = torch.eye(K, dtype=torch.bfloat16)[:64]
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float32)
    out = matmul(x.to(device), v, None, precision_config=pc)
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    deq = upcast_from_mxfp_ref(rv, rs, torch.float32, axis=0)
    assert torch.equal(out.cpu(), deq[:64])
    vz = torch.zeros_like(v)
    bias = torch.randn(N)
    betas, gammas = torch.rand(64) + 0.5, torch.rand(64) + 0.5
    out = matmul(x.to(device), vz, bias.to(device), precision_config=pc, betas=betas.to(device), gammas=gammas.to(device))
    torch.testing.assert_close(out.cpu(), bias[None] * betas[:, None] * gammas[:, None], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("block_m", [None, 16, 32, 64, 128])
@pytest.mark.parametrize("do_gather,do_scatter,do_gamma,act", [(False, False, False, False), (True, False, False, True),
                                                                (True, True, True, False), (False, True, True, True)])
def test_ragged(block_m, do_gather, do_scatter, do_gamma, act, device):
    torch.manual_seed(0)
    E, K, N, M = 9, 320, 392, 700
    sizes = torch.tensor([0, 5, 130, 16, 1, 257, 64, 200, 27], dtype=torch.int32)
    assert int(sizes.sum()) == M
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    gather = torch.randint(0, M, (M, ), dtype=torch.int32) if do_gather else None
    scatter = torch.randperm(M, dtype=torch.int32) if do_scatter else None
    if do_scatter:
        scatter[::13] = -1
    gammas = 2.0**torch.randint(-5, 0, (M, )).float() if do_gamma else None
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    dev = lambda t: None if t is None else t.to(device)
    fa = swiglu_act(1.702, 7.0) if act else None
    out_init = torch.zeros((M, N // 2 if act else N), dtype=torch.bfloat16, device=device)
    with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
        out = matmul(dev(x), v, dev(bias), md, gather_indx=dev(gather), scatter_indx=dev(scatter), precision_config=pc,
                     gammas=dev(gammas), fused_activation=fa, c=out_init)
    kw = dict(slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=rs, gammas=gammas)
    # kernel order: activation on the float32 accumulator (strict tolerance)
    ref = MR.matmul_ref(x, rv, bias, fused_swiglu=(1.702, 7.0) if act else None, **kw)
    check(out, ref)
    if act and not do_gamma:
        # order of the reference's test: bf16 result, then swiglu (its own error measure)
        ref2 = MR.swiglu_ref(MR.matmul_ref(x, rv, bias, **kw), 1.702, 7.0)
        assert_close(ref2, out.cpu(), maxtol=3e-2, verbose=False)


def test_moe_up_projection_small(device):
    """Config-3-shaped pipeline at reduced size: routing -> gather -> grouped GEMM + SwiGLU."""
    torch.manual_seed(0)
    T, E, k, H, N = 512, 16, 4, 2880, 768
    logits = torch.randn(T, E)
    x = torch.randn(T, H).to(torch.bfloat16)
    w = torch.randn(E, H, N) * 0.02
    bias = (torch.randn(E, N) * 0.01).to(torch.bfloat16)
    v, s, rv, rs = quantize_w(w, device)
    r = routing(logits.to(device), k)
    rr = RR.routing_ref(logits, k)
    assert torch.equal(r.gather_indx.cpu(), rr["gather_indx"])
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    out = matmul(x.to(device), v, bias.to(device), r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc,
                 fused_activation=swiglu_act(1.702, 7.0))
    kw = dict(slice_sizes=rr["col_sum"], gather_indx=rr["gather_indx"], b_mx_scale=rs)
    ref = MR.matmul_ref(x, rv, bias, fused_swiglu=(1.702, 7.0), **kw)
    assert tuple(out.shape) == (T * k, N // 2)
    check(out, ref)
    ref2 = MR.swiglu_ref(MR.matmul_ref(x, rv, bias, **kw), 1.702, 7.0)
    assert_close(ref2, out.cpu(), maxtol=3e-2, verbose=False)


def test_batched(device):
    torch.manual_seed(2)
    B, M, K, N = 3, 40, 128, 320
    x = torch.randn(B, M, K).to(torch.bfloat16)
    w = torch.randn(B, K, N) * 0.05
    v, s, rv, rs = quantize_w(w, device)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    out = matmul(x.to(device), v, None, precision_config=pc)
    ref = MR.matmul_ref(x, rv, None, b_mx_scale=rs)
    assert tuple(out.shape) == (B, M, N)
    check(out, ref)


def test_empty(device):
    w = torch.zeros((64, 32), dtype=torch.uint8, device=device).T  # [K/2=32, N=64], unit stride along K
    s = torch.zeros((64, 2), dtype=torch.uint8, device=device).T
    out = matmul(torch.empty((0, 64), dtype=torch.bfloat16, device=device), w, None,
                 precision_config=PrecisionConfig(b_mx_scale=s, b_microblock_size=32))
    assert tuple(out.shape) == (0, 64)


# ---------------------------------------------------------------------------- fp8 activations (scaled MFMA)


def to_fp8(x0, fp8=torch.float8_e4m3fn):
    """Per-tensor flex quantisation as in BASELINE config 5: s = amax / 448, x = (x0 / s) -> e4m3 (or e5m2: the
    activation type of most fp8 cases of the reference, tests/test_matmul.py:150-196)."""
    s = x0.abs().max() / 448.0
    return (x0 / s).to(fp8), s.reshape(1).float()


def fp8_pc(s_w, x_scale, device, out_dtype, fp8=torch.float8_e4m3fn):
    flex = FlexCtx(lhs_data=InFlexData(dtype=fp8, scale=x_scale.to(device)))
    return PrecisionConfig(b_mx_scale=s_w, b_microblock_size=32, flex_ctx=flex, out_dtype=out_dtype)


@pytest.mark.parametrize("M,K,N", [(256, 2048, 512), (16, 64, 64), (33, 96, 200), (130, 192, 520), (1, 32, 16),
                                   (128, 2880, 256)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_fp8_dense(M, K, N, out_dtype, fp8, device):
    torch.manual_seed(0)
    x8, xs = to_fp8(torch.randn(M, K), fp8)
    w = torch.randn(K, N) * 0.02
    bias = torch.randn(N) * 0.1
    v, s, rv, rs = quantize_w(w, device)
    out = matmul(x8.to(device), v, bias.to(device), precision_config=fp8_pc(s, xs, device, out_dtype, fp8))
    ref = MR.matmul_ref(x8, rv, bias, b_mx_scale=rs, a_flex_scale=xs)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    check(out, ref.to(out_dtype))


@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_fp8_one_hot_rows_are_exact(fp8, device):
    """x = one-hot rows (1.0 is exact in e4m3): the scaled MFMA must return the dequantised weight rows bit for
    bit, which pins the K order of both operands and the scale-byte selection."""
    torch.manual_seed(1)
    K, N = 256, 256
    w = torch.randn(K, N)
    v, s, rv, rs = quantize_w(w, device)
    x8 = torch.eye(K)[:160].to(fp8)
    one = torch.ones(1)
    out = matmul(x8.to(device), v, None, precision_config=fp8_pc(s, one, device, torch.float32, fp8))
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    deq = upcast_from_mxfp_ref(rv, rs, torch.float32, axis=0)
    assert torch.equal(out.cpu(), deq[:160])


@pytest.mark.parametrize("block_m", [None, 16, 32, 64, 128])
@pytest.mark.parametrize("do_gather,do_scatter,do_gamma,act", [(False, False, False, False), (True, False, False, True),
                                                                (False, True, True, False)])
@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_fp8_ragged(block_m, do_gather, do_scatter, do_gamma, act, fp8, device):
    torch.manual_seed(0)
    E, K, N, M = 9, 320, 392, 700
    sizes = torch.tensor([0, 5, 130, 16, 1, 257, 64, 200, 27], dtype=torch.int32)
    x8, xs = to_fp8(torch.randn(M, K), fp8)
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    gather = torch.randint(0, M, (M, ), dtype=torch.int32) if do_gather else None
    scatter = torch.randperm(M, dtype=torch.int32) if do_scatter else None
    if do_scatter:
        scatter[::13] = -1
    gammas = 2.0**torch.randint(-5, 0, (M, )).float() if do_gamma else None
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    dev = lambda t: None if t is None else t.to(device)
    fa = swiglu_act(1.702, 7.0) if act else None
    out_init = torch.zeros((M, N // 2 if act else N), dtype=torch.bfloat16, device=device)
    with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
        out = matmul(dev(x8), v, dev(bias), md, gather_indx=dev(gather), scatter_indx=dev(scatter),
                     precision_config=fp8_pc(s, xs, device, torch.bfloat16, fp8), gammas=dev(gammas), fused_activation=fa,
                     c=out_init)
    ref = MR.matmul_ref(x8, rv, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=rs,
                        a_flex_scale=xs, gammas=gammas, fused_swiglu=(1.702, 7.0) if act else None)
    check(out, ref.to(torch.bfloat16))


@pytest.mark.parametrize("block_m", [32, 64, 128])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float8_e4m3fn])
@pytest.mark.parametrize("K", [4608, 6432])
def test_fp8_ragged_long_k_strided_scales(block_m, out_dtype, K, device):
    """K = 4608 with strided scales: a tile's scales (256 columns x 144 bytes) no longer fit LDS beside the pipeline of a
    128-row block, so they travel with the weight stages (byte-sized copies); smaller blocks still stage them.
    K = 6432 (201 groups): no block size can stage them, so row blocks of up to 64 rows run the paired ring loop with
    strided scales, over an odd number of stages (51) whose last holds a single group.  Also the plain
    float8_e4m3fn output of fp8-row kernels (the rows the next matmul of a layer consumes)."""
    torch.manual_seed(3)
    E, N, M = 3, 264, 300
    sizes = torch.tensor([130, 0, 170], dtype=torch.int32)
    x8, xs = to_fp8(torch.randn(M, K), torch.float8_e4m3fn)
    w = torch.randn(E, K, N) * 0.02
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    gammas = 2.0**torch.randint(-3, 0, (M, )).float()
    with scoped_opt_flags_constraints({"block_m": block_m}):
        out = matmul(x8.to(device), v, bias.to(device), md, gammas=gammas.to(device),
                     precision_config=fp8_pc(s, xs, device, out_dtype, torch.float8_e4m3fn))
    ref = MR.matmul_ref(x8, rv, bias, slice_sizes=sizes, b_mx_scale=rs, a_flex_scale=xs, gammas=gammas)
    assert out.dtype == out_dtype
    if out_dtype == torch.bfloat16:
        check(out, ref.to(torch.bfloat16))
    else:
        # one fp8 step (2^-3 relative) around the float32 result
        torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=0.0725, atol=2e-2)


@pytest.mark.parametrize("kind", ["tiled_bf16", "stream_bf16", "tiled_fp8"])
def test_zero_scale_bytes_with_nonzero_codes(kind, device):
    """A checkpoint prepared elsewhere may hold e8m0 bytes of 0 next to non-zero codes (downcast_to_mxfp never writes
    that).  The reference multiplies such a group by +0.0; the conversion instructions multiply by 2^-127, i.e. the group
    contributes at most 6 * 2^-127 per element: the outputs agree with the oracle to far below the tolerance."""
    torch.manual_seed(11)
    M, K, N = (8, 256, 64) if kind == "stream_bf16" else (150, 256, 264)
    w = torch.randn(1, K, N) * 0.05
    v, s, rv, rs = quantize_w(w, device)
    rs = rs.clone()
    rs[0, ::3, ::2] = 0          # every third group of every second column
    s = rs.to(device)
    assert int((rv[0, :16, 0] != 0).sum()) > 0  # the zeroed groups do hold non-zero codes
    bias = torch.randn(1, N)
    sizes = torch.tensor([M], dtype=torch.int32)
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    if kind == "tiled_fp8":
        x8, xs = to_fp8(torch.randn(M, K))
        out = matmul(x8.to(device), v, bias.to(device), md, precision_config=fp8_pc(s, xs, device, torch.bfloat16))
        ref = MR.matmul_ref(x8, rv, bias, slice_sizes=sizes, b_mx_scale=rs, a_flex_scale=xs).to(torch.bfloat16)
    else:
        x = torch.randn(M, K).to(torch.bfloat16)
        out = matmul(x.to(device), v, bias.to(device), md, precision_config=PrecisionConfig(b_mx_scale=s, b_microblock_size=32))
        ref = MR.matmul_ref(x, rv, bias, slice_sizes=sizes, b_mx_scale=rs)
    assert torch.isfinite(out.float()).all()
    check(out, ref)


def test_moe_down_projection_and_combine_small(device):
    """Config-5-shaped pipeline at reduced size: expert-sorted fp8 rows -> grouped GEMM * gate weights ->
    scatter to (token, slot) order -> top-k combine."""
    from triton_amd.reduce import reduce
    torch.manual_seed(0)
    T, E, k, H = 256, 8, 4, 2880
    N = 384
    logits = torch.randn(T, E)
    r = routing(logits.to(device), k)
    rr = RR.routing_ref(logits, k)
    x8, xs = to_fp8(torch.randn(T * k, H))
    w = torch.randn(E, H, N) * 0.02
    bias = (torch.randn(E, N) * 0.01).to(torch.bfloat16)
    v, s, rv, rs = quantize_w(w, device)
    gam = r.expert_sorted_gate_weights
    gam_ref = rr["vals"].flatten()[rr["col_sorted_indx"].long()]
    torch.testing.assert_close(gam.cpu(), gam_ref, rtol=1e-5, atol=1e-7)  # softmax values: exp is not bit-pinned
    gam_ref = gam.cpu()
    y = matmul(x8.to(device), v, bias.to(device), r.ragged_metadata, scatter_indx=r.scatter_indx,
               precision_config=fp8_pc(s, xs, device, torch.bfloat16), gammas=gam)
    y_ref = MR.matmul_ref(x8, rv, bias, slice_sizes=rr["col_sum"], scatter_indx=rr["scatter_indx"], b_mx_scale=rs,
                          a_flex_scale=xs, gammas=gam_ref).to(torch.bfloat16)
    check(y, y_ref)
    z, _ = reduce(y.view(T, k, N), dim=1)
    z_ref = MR.reduce_ref(y.cpu().view(T, k, N), 1)
    assert torch.equal(z.cpu(), z_ref)  # fixed summation order: the combine is bit-exact given y


# ---------------------------------------------------------------------------- decode: weight-streaming kernel


@pytest.mark.parametrize("K", [64, 320, 1024, 2048, 2880, 4096])
@pytest.mark.parametrize("act,bias_dtype,xdtype", [(True, torch.bfloat16, torch.bfloat16), (False, torch.float32, torch.bfloat16),
                                                   (True, torch.float16, torch.float16)])
def test_decode_row_blocks_of_16(K, act, bias_dtype, xdtype, device):
    """Few rows per expert, N a multiple of 16, K dense per column: the streaming kernel (split-K over the
    waves, linear weight images) against the oracle; gather, scatter with dropped rows, gate weights."""
    torch.manual_seed(K)
    E, N = 7, 608
    sizes = torch.tensor([3, 0, 1, 16, 5, 21, 2], dtype=torch.int32)  # 21 rows: two row blocks for one expert
    M = int(sizes.sum())
    x = torch.randn(M + 5, K).to(xdtype)
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N).to(bias_dtype)
    v, s, rv, rs = quantize_w(w, device)
    gather = torch.randint(0, M + 5, (M, ), dtype=torch.int32)
    scatter = torch.randperm(M, dtype=torch.int32)
    scatter[::7] = -1
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    out_init = torch.zeros((M, N // 2 if act else N), dtype=xdtype, device=device)
    with scoped_opt_flags_constraints({"block_m": 16}):
        out = matmul(x.to(device), v, bias.to(device), md, gather_indx=gather.to(device), scatter_indx=scatter.to(device),
                     precision_config=pc, gammas=gammas.to(device), fused_activation=swiglu_act(1.702, 7.0) if act else None,
                     c=out_init)
    ref = MR.matmul_ref(x, rv, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=rs,
                        gammas=gammas, fused_swiglu=(1.702, 7.0) if act else None)
    check(out, ref)


def test_decode_shape_of_the_baseline(device):
    """Config 4 at reduced expert count: T=64 tokens, top-4 of 16 experts, K=2880, N=5760, bias + SwiGLU."""
    torch.manual_seed(0)
    T, E, k, H, N = 64, 16, 4, 2880, 5760
    logits = torch.randn(T, E)
    x = torch.randn(T, H).to(torch.bfloat16)
    bias = (torch.randn(E, N) * 0.01).to(torch.bfloat16)
    v = torch.empty((E, H // 2, N), dtype=torch.uint8, device=device).transpose(1, 2).contiguous().transpose(1, 2)
    s = torch.empty((E, H // 32, N), dtype=torch.uint8, device=device).transpose(1, 2).contiguous().transpose(1, 2)
    rv, rs = torch.empty_like(v, device="cpu"), torch.empty_like(s, device="cpu")
    for e in range(E):
        ve, se, rve, rse = quantize_w(torch.randn(1, H, N) * 0.02, device)
        v[e].copy_(ve[0]), s[e].copy_(se[0]), rv[e].copy_(rve[0]), rs[e].copy_(rse[0])
    r = routing(logits.to(device), k)
    rr = RR.routing_ref(logits, k)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    with scoped_opt_flags_constraints({"block_m": 16}):
        out = matmul(x.to(device), v, bias.to(device), r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc,
                     fused_activation=swiglu_act(1.702, 7.0))
    ref = MR.matmul_ref(x, rv, bias, slice_sizes=rr["col_sum"], gather_indx=rr["gather_indx"], b_mx_scale=rs,
                        fused_swiglu=(1.702, 7.0))
    check(out, ref)


# ---------------------------------------------------------------------------- flexpoint (fp8) output


@pytest.mark.parametrize("fp8,top", [(torch.float8_e4m3fn, 6.0), (torch.float8_e5m2, 11.0)])
def test_fp8_output_conversion_is_exact(fp8, top, device):
    """One-hot activations times a per-row gate weight give single float32 products deq(W)[k, n] * gamma[r]: the
    fp8 output must equal torch's own float32 -> fp8 cast of them bit for bit (round to nearest even, subnormals,
    beyond the range NaN for e4m3fn and infinity for e5m2 without saturation, the largest finite value with it)."""
    from triton_amd.matmul import OutFlexData
    torch.manual_seed(0)
    K, N, M = 64, 256, 64
    w = torch.randn(K, N) * 4
    v, s, rv, rs = quantize_w(w, device)
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    deq = upcast_from_mxfp_ref(rv, rs, torch.float32, axis=0)
    x = torch.eye(K, dtype=torch.bfloat16)[:M]
    gammas = torch.exp(torch.linspace(-12 - top / 2, top, M)).float()
    max_q = torch.finfo(fp8).max
    for saturate in (False, True):
        actual = torch.zeros(1, device=device)
        flex = FlexCtx(out_data=OutFlexData(fp8, torch.ones(1, device=device), actual, None))
        pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32, out_dtype=fp8, flex_ctx=flex,
                             flexpoint_saturate_inf=saturate)
        out = matmul(x.to(device), v, None, precision_config=pc, gammas=gammas.to(device))
        assert out.dtype == fp8
        prod = deq[:M] * gammas[:, None]
        assert prod.abs().max() > 1.2 * max_q  # the range is exceeded somewhere
        want = (prod.clamp(-max_q, max_q) if saturate else prod).to(fp8)
        # a -0.0 weight summed with the +0.0 products of the other K positions is +0.0: ignore the sign of zero
        pos_zero = lambda t: torch.where(t == 0x80, torch.zeros_like(t), t)
        assert torch.equal(pos_zero(out.cpu().view(torch.uint8)), pos_zero(want.view(torch.uint8)))
        assert actual.item() == pytest.approx(float(prod.abs().max()) / max_q, rel=1e-6)


@pytest.mark.parametrize("block_m", [16, 128])
@pytest.mark.parametrize("act", [False, True])
def test_fp8_output_with_expected_scale(block_m, act, device):
    """FC1-style problem emitting fp8 with a flexpoint scale: values = result / expected_scale cast to e4m3, and
    the actual scale is max|result| / 448 (reference: float_to_flex / compute_actual_scale)."""
    from triton_amd.matmul import OutFlexData
    torch.manual_seed(1)
    E, K, N = 5, 320, 384
    sizes = torch.tensor([3, 0, 16, 140, 9], dtype=torch.int32)
    M = int(sizes.sum())
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    expected = torch.tensor([0.03125], device=device)
    actual = torch.zeros(1, device=device)
    flex = FlexCtx(out_data=OutFlexData(torch.float8_e4m3fn, expected, actual, None))
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float8_e4m3fn, flex_ctx=flex,
                         flexpoint_saturate_inf=True)
    with scoped_opt_flags_constraints({"block_m": block_m}):
        out = matmul(x.to(device), v, bias.to(device), md, precision_config=pc,
                     fused_activation=swiglu_act(1.702, 7.0) if act else None)
    ref32 = MR.matmul_ref(x.float(), rv, bias, slice_sizes=sizes, b_mx_scale=rs, fused_swiglu=(1.702, 7.0) if act else None)
    want = (ref32 / 0.03125).clamp(-448, 448)
    got = out.float().cpu()
    # fp8 has 3 mantissa bits: one step of the result grid is 2^-3 relative; allow one step plus the GEMM tolerance
    assert ((got - want).abs() <= 0.13 * want.abs() + 0.02 / 0.03125).all()
    assert_close(want.to(torch.float8_e4m3fn).float(), got, maxtol=7e-2, rmstol=2e-2, verbose=False)
    assert actual.item() == pytest.approx(MR.actual_scale_ref(ref32, torch.float8_e4m3fn).item(), rel=2e-3)


def test_moe_mlp_chain_with_fp8_intermediate(device):
    """routing -> FC1 (gather, bias, SwiGLU) emitting fp8 with a flexpoint scale -> FC2 consuming those fp8 rows
    with the same scale (gate weights, scatter) -> top-k combine; against the oracle chained the same way."""
    from triton_amd.matmul import OutFlexData
    from triton_amd.reduce import reduce
    torch.manual_seed(0)
    T, E, k, H, I = 192, 8, 2, 256, 512
    logits = torch.randn(T, E)
    x = torch.randn(T, H).to(torch.bfloat16)
    w1 = torch.randn(E, H, 2 * I) * 0.05
    w2 = torch.randn(E, I, H) * 0.05
    b1, b2 = torch.randn(E, 2 * I) * 0.1, torch.randn(E, H) * 0.1
    v1, s1, rv1, rs1 = quantize_w(w1, device)
    v2, s2, rv2, rs2 = quantize_w(w2, device)
    r = routing(logits.to(device), k)
    rr = RR.routing_ref(logits, k)
    mid_scale = torch.tensor([1.0 / 64], device=device)
    actual = torch.zeros(1, device=device)
    pc1 = PrecisionConfig(b_mx_scale=s1, b_microblock_size=32, out_dtype=torch.float8_e4m3fn, flexpoint_saturate_inf=True,
                          flex_ctx=FlexCtx(out_data=OutFlexData(torch.float8_e4m3fn, mid_scale, actual, None)))
    h = matmul(x.to(device), v1, b1.to(device), r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc1,
               fused_activation=swiglu_act(1.702, 7.0))
    assert h.dtype == torch.float8_e4m3fn and tuple(h.shape) == (T * k, I)
    pc2 = PrecisionConfig(b_mx_scale=s2, b_microblock_size=32, out_dtype=torch.bfloat16,
                          flex_ctx=FlexCtx(lhs_data=InFlexData(torch.float8_e4m3fn, mid_scale)))
    gam = r.expert_sorted_gate_weights
    y = matmul(h, v2, b2.to(device), r.ragged_metadata, scatter_indx=r.scatter_indx, precision_config=pc2, gammas=gam)
    z, _ = reduce(y.view(T, k, H), dim=1)
    # oracle: same chain, the fp8 rounding of the intermediate included (taken from the kernel's own fp8 rows, which
    # are checked against the float32 oracle first)
    h_ref32 = MR.matmul_ref(x.float(), rv1, b1, slice_sizes=rr["col_sum"], gather_indx=rr["gather_indx"], b_mx_scale=rs1,
                            fused_swiglu=(1.702, 7.0))
    want_h = (h_ref32 * 64).clamp(-448, 448)
    assert ((h.float().cpu() - want_h).abs() <= 0.13 * want_h.abs() + 0.64).all()
    assert actual.item() == pytest.approx(MR.actual_scale_ref(h_ref32, torch.float8_e4m3fn).item(), rel=2e-3)
    y_ref = MR.matmul_ref(h.cpu(), rv2, b2, slice_sizes=rr["col_sum"], scatter_indx=rr["scatter_indx"], b_mx_scale=rs2,
                          a_flex_scale=mid_scale.cpu(), gammas=gam.cpu()).to(torch.bfloat16)
    check(y, y_ref)
    assert torch.equal(z.cpu(), MR.reduce_ref(y.cpu().view(T, k, H), 1))


# ---------------------------------------------------------------------------- unquantised 16-bit weights


@pytest.mark.parametrize("M,K,N", [(256, 2880, 128), (16, 64, 64), (33, 96, 200), (130, 192, 520), (1, 8, 8), (300, 2048, 1024)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("k_contiguous", [False, True])
def test_dense_16bit_weights(M, K, N, dtype, k_contiguous, device):
    """(256, 2880, 128) is the gate matmul of the MoE block (hidden -> expert logits)."""
    torch.manual_seed(0)
    x = torch.randn(M, K).to(dtype)
    w = (torch.randn(K, N) * 0.05).to(dtype)
    bias = torch.randn(N)
    wd = w.to(device)
    if k_contiguous:
        wd = wd.T.contiguous().T  # same values, unit stride along K
        assert wd.stride() == (1, K)
    out = matmul(x.to(device), wd, bias.to(device))
    ref = MR.matmul_ref(x, w, bias)
    assert out.dtype == dtype and tuple(out.shape) == (M, N)
    check(out, ref)


@pytest.mark.parametrize("M,K,N", [(2048, 5760, 128), (100, 136, 40), (17, 8, 100), (5, 2888, 128), (64, 64, 8), (333, 4096, 72)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("out_f32", [False, True])
def test_narrow_dense_product(M, K, N, dtype, out_f32, device):
    """N <= 128 goes to the kernel without LDS staging (16 rows x 64 columns per workgroup, K split over the waves):
    ragged edges in M, N and K, bias on and off, float32 output, both storage orders of the weights.
    (2048, 5760, 128) is the gate matmul of the reference's bench_mlp."""
    torch.manual_seed(M + N)
    x = torch.randn(M, K).to(dtype)
    w = (torch.randn(K, N) * 0.05).to(dtype)
    bias = torch.randn(N) if N != 40 else None
    pc = PrecisionConfig(out_dtype=torch.float32) if out_f32 else None
    for wd in (w.to(device), w.to(device).T.contiguous().T):
        out = matmul(x.to(device), wd, None if bias is None else bias.to(device), precision_config=pc)
        ref = MR.matmul_ref(x, w, bias)
        assert out.dtype == (torch.float32 if out_f32 else dtype) and tuple(out.shape) == (M, N)
        check(out, ref if not out_f32 else (x.float() @ w.float() + (0 if bias is None else bias)))


@pytest.mark.parametrize("block_m", [None, 16, 64])
@pytest.mark.parametrize("act", [False, True])
def test_ragged_16bit_weights(block_m, act, device):
    torch.manual_seed(1)
    E, K, N, M = 6, 320, 392, 500
    sizes = torch.tensor([0, 5, 130, 16, 249, 100], dtype=torch.int32)
    x = torch.randn(M + 3, K).to(torch.bfloat16)
    w = (torch.randn(E, K, N) * 0.05).to(torch.bfloat16)
    bias = torch.randn(E, N)
    gather = torch.randint(0, M + 3, (M, ), dtype=torch.int32)
    scatter = torch.randperm(M, dtype=torch.int32)
    scatter[::11] = -1
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    out_init = torch.zeros((M, N // 2 if act else N), dtype=torch.bfloat16, device=device)
    with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
        out = matmul(x.to(device), w.to(device), bias.to(device), md, gather_indx=gather.to(device),
                     scatter_indx=scatter.to(device), gammas=gammas.to(device),
                     fused_activation=swiglu_act(1.702, 7.0) if act else None, c=out_init)
    ref = MR.matmul_ref(x, w, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, gammas=gammas,
                        fused_swiglu=(1.702, 7.0) if act else None)
    check(out, ref)


# ---------------------------------------------------------------------------- pre-shuffled (CDNA4) weight scales


def preshuffle(s):
    """Scales as downcast_to_mxfp returns them -> the CDNA4 scale layout, checked against the oracle's bytes."""
    import numpy as np
    from oracle import layout_ref as LR
    from triton_amd.tensor import convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import CDNA4MXScaleLayout
    t = convert_layout(wrap_torch_tensor(s), CDNA4MXScaleLayout())
    d = t.storage.data
    flat = d.transpose(-1, -2).reshape(d.shape[0], d.shape[1] * d.shape[2]).cpu().numpy()
    assert np.array_equal(flat, LR.cdna4_swizzle_ref(s.cpu().contiguous().numpy()))
    return t


@pytest.mark.parametrize("M,K,N", [(256, 2048, 4096), (16, 64, 64), (33, 96, 208), (130, 192, 528), (1, 32, 16),
                                   (70, 2880, 5760 // 8)])
@pytest.mark.parametrize("fp8", [False, True])
def test_dense_with_preshuffled_scales(M, K, N, fp8, device):
    """The same kernel, same arithmetic: results must equal the strided-scale ones bit for bit, and match the oracle."""
    torch.manual_seed(0)
    w = torch.randn(K, N) * 0.02
    bias = (torch.randn(N) * 0.01).to(torch.bfloat16)
    v, s, rv, rs = quantize_w(w, device)
    if fp8:
        x, x_scale = to_fp8(torch.randn(M, K))
        flex = FlexCtx(lhs_data=InFlexData(dtype=torch.float8_e4m3fn, scale=x_scale.to(device)))
        mk = lambda sc: PrecisionConfig(b_mx_scale=sc, b_microblock_size=32, flex_ctx=flex, out_dtype=torch.bfloat16)
        ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs, a_flex_scale=x_scale).to(torch.bfloat16)
    else:
        x = torch.randn(M, K).to(torch.bfloat16)
        mk = lambda sc: PrecisionConfig(b_mx_scale=sc, b_microblock_size=32)
        ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs)
    out_s = matmul(x.to(device), v, bias.to(device), precision_config=mk(s))
    out_p = matmul(x.to(device), v, bias.to(device), precision_config=mk(preshuffle(s)))
    assert torch.equal(out_p, out_s)
    check(out_p, ref)


@pytest.mark.parametrize("block_m", [None, 16, 32, 128])
@pytest.mark.parametrize("K,N", [(320, 400), (2880, 608), (4096, 96)])
@pytest.mark.parametrize("fp8", [False, True])
def test_ragged_with_preshuffled_scales(block_m, K, N, fp8, device):
    """Ragged, gather + scatter + gate weights + SwiGLU; block_m 16 with N % 16 == 0 runs the streaming kernel,
    whose units are halves of the 32-column scale blocks."""
    torch.manual_seed(1)
    E = 7
    sizes = torch.tensor([3, 0, 1, 16, 5, 140, 2], dtype=torch.int32)
    M = int(sizes.sum())
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    gather = torch.randint(0, M + 5, (M, ), dtype=torch.int32)
    scatter = torch.randperm(M, dtype=torch.int32)
    scatter[::7] = -1
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    kw = dict(slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=rs, gammas=gammas,
              fused_swiglu=(1.702, 7.0))
    if fp8:
        x, x_scale = to_fp8(torch.randn(M + 5, K))
        flex = FlexCtx(lhs_data=InFlexData(dtype=torch.float8_e4m3fn, scale=x_scale.to(device)))
        mk = lambda sc: PrecisionConfig(b_mx_scale=sc, b_microblock_size=32, flex_ctx=flex, out_dtype=torch.bfloat16)
        ref = MR.matmul_ref(x, rv, bias, a_flex_scale=x_scale, **kw).to(torch.bfloat16)
    else:
        x = torch.randn(M + 5, K).to(torch.bfloat16)
        mk = lambda sc: PrecisionConfig(b_mx_scale=sc, b_microblock_size=32)
        ref = MR.matmul_ref(x, rv, bias, **kw)
    outs = []
    for sc in (s, preshuffle(s)):
        out_init = torch.zeros((M, N // 2), dtype=torch.bfloat16, device=device)
        with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
            outs.append(matmul(x.to(device), v, bias.to(device), md, gather_indx=gather.to(device),
                               scatter_indx=scatter.to(device), precision_config=mk(sc), gammas=gammas.to(device),
                               fused_activation=swiglu_act(1.702, 7.0), c=out_init))
    assert torch.equal(outs[1], outs[0])
    check(outs[1], ref)


# ---------------------------------------------------------------------------- MXFP8 activations (block-scaled fp8 rows)


def quantize_x_mxfp8(x0, device):
    """fp32 [.., K] -> (e4m3 values, e8m0 scales per 32 along K) on the GPU, checked against the oracle."""
    xq, xs = downcast_to_mxfp(x0.to(device), torch.float8_e4m3fn, axis=-1)
    rq, rs = downcast_to_mxfp_ref(x0, torch.float8_e4m3fn, axis=-1)
    assert torch.equal(xq.cpu().view(torch.uint8), rq.contiguous().view(torch.uint8)) and torch.equal(xs.cpu(), rs)
    return xq, xs, rq.contiguous(), rs.contiguous()


@pytest.mark.parametrize("M,K,N", [(256, 2048, 512), (16, 64, 64), (33, 96, 208), (130, 192, 528), (70, 2880, 720)])
@pytest.mark.parametrize("out_dtype", [None, torch.float32])
def test_mxfp8_activations_dense(M, K, N, out_dtype, device):
    torch.manual_seed(0)
    x0 = torch.randn(M, K) * torch.exp(torch.randn(M, K // 32).repeat_interleave(32, dim=1) * 2)  # block-wise dynamic range
    w = torch.randn(K, N) * 0.02
    bias = (torch.randn(N) * 0.01).to(torch.bfloat16)
    v, s, rv, rs = quantize_w(w, device)
    xq, xs, rq, rxs = quantize_x_mxfp8(x0, device)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32, out_dtype=out_dtype)
    out = matmul(xq, v, bias.to(device), precision_config=pc)
    ref = MR.matmul_ref(rq, rv, bias, a_mx_scale=rxs, b_mx_scale=rs)
    assert out.dtype == (out_dtype or torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL * float(ref.float().abs().max()) / 4 + ATOL)
    # doubling every block scale of the activations doubles the linear part exactly
    pc32 = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float32)
    pc32b = PrecisionConfig(a_mx_scale=xs + 1, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float32)
    assert torch.equal(matmul(xq, v, None, precision_config=pc32b), 2 * matmul(xq, v, None, precision_config=pc32))


@pytest.mark.parametrize("block_m", [None, 16, 64, 128])
@pytest.mark.parametrize("cdna4_scales", [False, True])
def test_mxfp8_activations_ragged(block_m, cdna4_scales, device):
    """Gather, scatter with dropped rows, gate weights, SwiGLU; the activation scales follow the gathered rows."""
    torch.manual_seed(1)
    E, K, N = 7, 320, 400
    sizes = torch.tensor([3, 0, 1, 16, 5, 140, 2], dtype=torch.int32)
    M = int(sizes.sum())
    x0 = torch.randn(M + 5, K) * torch.exp(torch.randn(M + 5, K // 32).repeat_interleave(32, dim=1))
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    xq, xs, rq, rxs = quantize_x_mxfp8(x0, device)
    gather = torch.randint(0, M + 5, (M, ), dtype=torch.int32)
    scatter = torch.randperm(M, dtype=torch.int32)
    scatter[::7] = -1
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=preshuffle(s) if cdna4_scales else s,
                         b_microblock_size=32)
    out_init = torch.zeros((M, N // 2), dtype=torch.bfloat16, device=device)
    with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
        out = matmul(xq, v, bias.to(device), md, gather_indx=gather.to(device), scatter_indx=scatter.to(device),
                     precision_config=pc, gammas=gammas.to(device), fused_activation=swiglu_act(1.702, 7.0), c=out_init)
    ref = MR.matmul_ref(rq, rv, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, a_mx_scale=rxs,
                        b_mx_scale=rs, gammas=gammas, fused_swiglu=(1.702, 7.0))
    check(out, ref)


# ---------------------------------------------------------------------------- weights in the kernels' block layout


@pytest.mark.parametrize("kind", ["tiled_bf16", "stream_bf16", "tiled_fp8", "k_groups"])
def test_block_layout_gives_the_same_bits(kind, device):
    """The 4 KB blocks hold a wave's LDS image as it is: the kernels do the same arithmetic in the same order from either
    layout, so the outputs are bit for bit the same (K and N ragged against the blocks: 2880 = 22.5 x 128, 400 = 6.25 x 64)."""
    torch.manual_seed(5)
    E, K, N = 4, 2880, 400
    rows = {"tiled_bf16": [150, 0, 33, 7], "stream_bf16": [3, 0, 9, 1], "tiled_fp8": [150, 0, 33, 7], "k_groups": [30, 20, 0, 5]}[kind]
    sizes = torch.tensor(rows, dtype=torch.int32)
    M = int(sizes.sum())
    w = torch.randn(E, K, N) * 0.03
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    if kind == "tiled_fp8":
        x8, xs = to_fp8(torch.randn(M, K), torch.float8_e4m3fn)
        x, pc = x8.to(device), fp8_pc(s, xs, device, torch.bfloat16, torch.float8_e4m3fn)
    else:
        x, pc = torch.randn(M, K).to(torch.bfloat16).to(device), PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    with scoped_opt_flags_constraints({"block_m": 32} if kind == "k_groups" else {}):
        y_strided = matmul(x, v, bias.to(device), md, precision_config=pc, fused_activation=swiglu_act(1.702, 7.0))
        y_blocks = matmul(x, in_blocks(v), bias.to(device), md, precision_config=pc, fused_activation=swiglu_act(1.702, 7.0))
    assert torch.equal(y_strided.view(torch.int16), y_blocks.view(torch.int16))


def test_metadata_made_for_fewer_rows_is_refused(device):
    """The kernels read as many schedule entries as the matmul's row count can need: ragged metadata made for fewer rows
    than the gathered activations have is refused on the host instead of being read past its end."""
    torch.manual_seed(0)
    E, K, N = 40, 64, 64
    sizes = torch.ones(E, dtype=torch.int32)
    md = make_ragged_tensor_metadata(sizes.to(device), E)           # 40 rows: at most 40 row blocks
    M = 2000                                                         # the matmul is given 2000 rows
    w = torch.randn(E, K, N) * 0.05
    v, s, _, _ = quantize_w(w, device)
    x = torch.randn(M, K).to(torch.bfloat16).to(device)
    with pytest.raises(ValueError, match="fewer rows"):
        matmul(x, v, None, md, precision_config=PrecisionConfig(b_mx_scale=s, b_microblock_size=32))


# ---------------------------------------------------------------------------- K groups (few 32-row tiles)


@pytest.mark.parametrize("K", [512, 1440, 2880])        # 4, 11.25 and 22.5 pairs of 128: two and four K groups, ragged ends
@pytest.mark.parametrize("mode", ["dense", "ragged", "batched"])
@pytest.mark.parametrize("cdna4", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_k_groups(K, mode, cdna4, dtype, device):
    """Row blocks of 32 with fewer tiles than CUs: the tile's K range is shared by groups of four waves whose partial
    sums meet in LDS.  The last group's part ends inside a pair (K = 1440, 2880) or holds no K at all."""
    torch.manual_seed(K)
    N = 400 if not cdna4 else 448
    E = 3
    act = mode != "batched"
    if mode == "dense":
        x, w, bias, sizes = torch.randn(70, K), torch.randn(K, N) * 0.05, torch.randn(N), None
    elif mode == "ragged":
        sizes = torch.tensor([33, 0, 30], dtype=torch.int32)
        x, w, bias = torch.randn(63, K), torch.randn(E, K, N) * 0.05, torch.randn(E, N)
    else:
        x, w, bias, sizes = torch.randn(E, 40, K), torch.randn(E, K, N) * 0.05, torch.randn(E, N), None
    x = x.to(dtype)
    v, s, rv, rs = quantize_w(w, device)
    pc = PrecisionConfig(b_mx_scale=preshuffle(s) if cdna4 else s, b_microblock_size=32)
    md = make_ragged_tensor_metadata(sizes.to(device), 63) if mode == "ragged" else None
    with scoped_opt_flags_constraints({"block_m": 32}):
        out = matmul(x.to(device), in_blocks(v) if cdna4 else v, bias.to(device), md, precision_config=pc,
                     fused_activation=swiglu_act(1.702, 7.0) if act else None)
    ref = MR.matmul_ref(x, rv, bias, slice_sizes=sizes, b_mx_scale=rs, fused_swiglu=(1.702, 7.0) if act else None)
    check(out, ref)


# ---------------------------------------------------------------------------- MXFP4 activations


def in_blocks(v):
    """MXFP4 codes as downcast_to_mxfp returns them -> the kernels' block layout."""
    return convert_layout(wrap_torch_tensor(v, dtype=FP4), CDNA4MXValueLayout())


def quantize_x_mxfp4(x0, device):
    """fp32 [.., K] -> (packed e2m1 codes [.., K/2], e8m0 scales per 32 along K) on the GPU, checked against the oracle."""
    xq, xs = downcast_to_mxfp(x0.to(device), torch.uint8, axis=-1)
    rq, rs = downcast_to_mxfp_ref(x0, torch.uint8, axis=-1)
    assert torch.equal(xq.cpu(), rq) and torch.equal(xs.cpu(), rs)
    return xq, xs, rq.contiguous(), rs.contiguous()


def test_widen_mxfp4_rows_every_code(device):
    """All 256 bytes: the widened pair of float8_e4m3fn numbers has the values of the two e2m1 codes, low nibble
    first, with the sign of zero kept; row strides honoured."""
    from triton_amd import _lib
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    src = torch.arange(256, dtype=torch.uint8).reshape(4, 64)
    wide = torch.zeros((4, 160), dtype=torch.uint8, device=device)
    d = src.to(device)
    rc = _lib.lib().tamd_widen_mxfp4_rows(_lib.ptr(d), 4, 64, 64, _lib.ptr(wide), 160, _lib.stream_ptr(d.device))
    assert rc == 0
    got = wide.cpu()
    assert torch.all(got[:, 128:] == 0)
    unit = torch.full((4, 4), 127, dtype=torch.uint8)                     # scale 2^0 for each 32 values
    want = upcast_from_mxfp_ref(src, unit, torch.float32, axis=-1)
    vals = got[:, :128].contiguous().view(torch.float8_e4m3fn).float()
    assert torch.equal(vals, want) and torch.equal(torch.signbit(vals), torch.signbit(want))


@pytest.mark.parametrize("swizzled", [False, True])
def test_mxfp4_activations_mxfp4_weights_plain(swizzled, device):
    """tests/test_matmul.py:234-235 of the reference: 256 x 256 x 256, both operands MXFP4, bf16 output."""
    torch.manual_seed(0)
    M = K = N = 256
    x0 = torch.randn(M, K) * torch.exp(torch.randn(M, K // 32).repeat_interleave(32, dim=1) * 2)
    w = torch.randn(K, N) * 0.02
    v, s, rv, rs = quantize_w(w, device)
    xq, xs, rq, rxs = quantize_x_mxfp4(x0, device)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=preshuffle(s) if swizzled else s,
                         b_microblock_size=32, out_dtype=torch.bfloat16)
    out = matmul(wrap_torch_tensor(xq, dtype=FP4), in_blocks(v) if swizzled else v, None, precision_config=pc)
    ref = MR.matmul_ref(rq, rv, None, a_mx_scale=rxs, b_mx_scale=rs)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL * float(ref.float().abs().max()) / 4 + ATOL)
    # the raw uint8 tensor is taken as packed codes too, and the product is linear in the block scales
    pc32 = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float32)
    pc32b = PrecisionConfig(a_mx_scale=xs + 1, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float32)
    y = matmul(xq, v, None, precision_config=pc32)
    assert torch.equal(matmul(xq, v, None, precision_config=pc32b), 2 * y)
    # e2m1 codes widened to fp8 are the same numbers: the MXFP8 path with the widened values gives the same bits
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    unit = torch.full_like(rxs, 127)
    x8 = upcast_from_mxfp_ref(rq, unit, torch.float32, axis=-1).to(torch.float8_e4m3fn).to(device)
    assert torch.equal(matmul(x8, v, None, precision_config=pc32), y)


@pytest.mark.parametrize("block_m", [None, 16, 64, 128])
@pytest.mark.parametrize("cdna4", [False, True])
def test_mxfp4_activations_mxfp4_weights_ragged(block_m, cdna4, device):
    """Gather, scatter with dropped rows, gate weights, SwiGLU on MXFP4 x MXFP4; with `cdna4` the weights are in the
    CDNA4 value layout and their scales in the CDNA4 scale layout."""
    torch.manual_seed(1)
    E, K, N = 7, 320, 400 if not cdna4 else 448
    sizes = torch.tensor([3, 0, 1, 16, 5, 140, 2], dtype=torch.int32)
    M = int(sizes.sum())
    x0 = torch.randn(M + 5, K) * torch.exp(torch.randn(M + 5, K // 32).repeat_interleave(32, dim=1))
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    xq, xs, rq, rxs = quantize_x_mxfp4(x0, device)
    gather = torch.randint(0, M + 5, (M, ), dtype=torch.int32)
    scatter = torch.randperm(M, dtype=torch.int32)
    scatter[::7] = -1
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=preshuffle(s) if cdna4 else s,
                         b_microblock_size=32)
    out_init = torch.zeros((M, N // 2), dtype=torch.bfloat16, device=device)
    with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
        out = matmul(xq, in_blocks(v) if cdna4 else v, bias.to(device), md, gather_indx=gather.to(device),
                     scatter_indx=scatter.to(device), precision_config=pc, gammas=gammas.to(device),
                     fused_activation=swiglu_act(1.702, 7.0), c=out_init)
    ref = MR.matmul_ref(rq, rv, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, a_mx_scale=rxs,
                        b_mx_scale=rs, gammas=gammas, fused_swiglu=(1.702, 7.0))
    check(out, ref)


def test_mxfp4_activations_prefill_shape(device):
    """The shape of the prefill up projection (K 2880, N 5760, 4 of 128 experts with rows; 1 row to several row
    blocks), MXFP4 activations against MXFP4 weights in the CDNA4 layouts."""
    torch.manual_seed(2)
    E, K, N = 6, 2880, 5760
    sizes = torch.tensor([300, 0, 1, 129, 64, 0], dtype=torch.int32)
    M = int(sizes.sum())
    x0 = torch.randn(M, K) * torch.exp(torch.randn(M, K // 32).repeat_interleave(32, dim=1))
    w = torch.randn(E, K, N) * 0.02
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    xq, xs, rq, rxs = quantize_x_mxfp4(x0, device)
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=preshuffle(s), b_microblock_size=32)
    out = matmul(xq, in_blocks(v), bias.to(device), md, precision_config=pc, fused_activation=swiglu_act(1.702, 7.0))
    ref = MR.matmul_ref(rq, rv, bias, slice_sizes=sizes, a_mx_scale=rxs, b_mx_scale=rs, fused_swiglu=(1.702, 7.0))
    check(out, ref)


@pytest.mark.parametrize("mode", ["ragged", "batched"])
@pytest.mark.parametrize("w_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("a_kind", ["mxfp4", "mxfp8"])
def test_mx_activations_16bit_weights(mode, w_dtype, a_kind, device):
    """tests/test_matmul.py:217-232 of the reference: 64 x 128 x 96, microscaled activations against unquantised
    bf16 / fp16 weights, bf16 output."""
    torch.manual_seed(3)
    M, N, K = 64, 128, 96
    E = 3
    quant = quantize_x_mxfp4 if a_kind == "mxfp4" else quantize_x_mxfp8
    if mode == "ragged":
        sizes = torch.tensor([20, 0, 44], dtype=torch.int32)
        x0 = torch.randn(M, K) * torch.exp(torch.randn(M, K // 32).repeat_interleave(32, dim=1))
    else:
        x0 = torch.randn(E, M, K) * torch.exp(torch.randn(E, M, K // 32).repeat_interleave(32, dim=2))
    w = (torch.randn(E, K, N) * 0.1).to(w_dtype)
    bias = torch.randn(E, N)
    xq, xs, rq, rxs = quant(x0, device)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, out_dtype=torch.bfloat16)
    if mode == "ragged":
        md = make_ragged_tensor_metadata(sizes.to(device), M)
        out = matmul(xq, w.to(device), bias.to(device), md, precision_config=pc)
        ref = MR.matmul_ref(rq, w, bias, slice_sizes=sizes, a_mx_scale=rxs)
    else:
        out = matmul(xq, w.to(device), bias.to(device), precision_config=pc)
        ref = MR.matmul_ref(rq, w, bias, a_mx_scale=rxs)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == tuple(ref.shape)
    check(out, ref)


@pytest.mark.parametrize("mode", ["ragged", "batched"])
def test_mxfp8_activations_mxfp8_weights(mode, device):
    """tests/test_matmul.py:214-216 of the reference: 300 x 400 x 416, both operands MXFP8."""
    torch.manual_seed(4)
    M, N, K = 300, 400, 416
    E = 3
    if mode == "ragged":
        sizes = torch.tensor([120, 0, 180], dtype=torch.int32)
        x0 = torch.randn(M, K) * torch.exp(torch.randn(M, K // 32).repeat_interleave(32, dim=1))
    else:
        x0 = torch.randn(E, M, K) * torch.exp(torch.randn(E, M, K // 32).repeat_interleave(32, dim=2))
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    wq, ws = downcast_to_mxfp(w.to(device), torch.float8_e4m3fn, axis=-2)
    rwq, rws = downcast_to_mxfp_ref(w, torch.float8_e4m3fn, axis=-2)
    assert torch.equal(wq.cpu().view(torch.uint8), rwq.contiguous().view(torch.uint8)) and torch.equal(ws.cpu(), rws)
    xq, xs, rq, rxs = quantize_x_mxfp8(x0, device)
    pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=ws, b_microblock_size=32,
                         out_dtype=torch.bfloat16)
    if mode == "ragged":
        md = make_ragged_tensor_metadata(sizes.to(device), M)
        out = matmul(xq, wq, bias.to(device), md, precision_config=pc)
        ref = MR.matmul_ref(rq, rwq, bias, slice_sizes=sizes, a_mx_scale=rxs, b_mx_scale=rws)
    else:
        out = matmul(xq, wq, bias.to(device), precision_config=pc)
        ref = MR.matmul_ref(rq, rwq, bias, a_mx_scale=rxs, b_mx_scale=rws)
    check(out, ref)


# ---------------------------------------------------------------------------- MXFP8 output (quantising epilogue)


def mxfp8_epilogue():
    from triton_amd.matmul import Epilogue
    return Epilogue(FnSpecs("QUANTIZE_MXFP8", None, (), ()), tuple(), tuple(), effective_itemsize=6.0)


@pytest.mark.parametrize("M,K,N", [(256, 2048, 512), (16, 64, 64), (33, 96, 208), (130, 192, 528)])
@pytest.mark.parametrize("act", [False, True])
def test_mxfp8_output_dense(M, K, N, act, device):
    """The quantised result must be bit for bit what downcast_to_mxfp makes of the float32 result of the same kernel
    (values and scale bytes), and dequantise to the oracle's result within the fp8 step."""
    torch.manual_seed(0)
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(K, N) * 0.02
    bias = torch.randn(N)
    v, s, rv, rs = quantize_w(w, device)
    fa = swiglu_act(1.702, 7.0) if act else None
    n_out = N // 2 if act else N
    y32 = matmul(x.to(device), v, bias.to(device), fused_activation=fa,
                 precision_config=PrecisionConfig(b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float32))
    c_scale = torch.zeros((M, -(-n_out // 32)), dtype=torch.uint8, device=device)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32, out_dtype=torch.float8_e4m3fn, c_mx_scale=c_scale)
    yq = matmul(x.to(device), v, bias.to(device), fused_activation=fa, precision_config=pc, epilogue=mxfp8_epilogue())
    assert yq.dtype == torch.float8_e4m3fn and tuple(yq.shape) == (M, n_out) and pc.c_microblock_size == 32
    pad = (-n_out) % 32
    y32p = torch.nn.functional.pad(y32.cpu(), (0, pad))
    want_v, want_s = downcast_to_mxfp_ref(y32p, torch.float8_e4m3fn, axis=-1)
    assert torch.equal(c_scale.cpu(), want_s)
    assert torch.equal(yq.cpu().view(torch.uint8), want_v[:, :n_out].contiguous().view(torch.uint8))
    ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs, fused_swiglu=(1.702, 7.0) if act else None).float()
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    deq = upcast_from_mxfp_ref(torch.nn.functional.pad(yq.cpu().view(torch.uint8), (0, pad)).view(torch.float8_e4m3fn),
                               c_scale.cpu(), torch.float32, axis=-1)[:, :n_out]
    gmax = torch.nn.functional.pad(ref.abs(), (0, pad)).reshape(M, -1, 32).amax(dim=-1).repeat_interleave(32, dim=1)[:, :n_out]
    assert torch.all((deq - ref).abs() <= gmax / 8 + 2e-2)  # e4m3 step at the top of a group is 1/16 of its maximum


@pytest.mark.parametrize("block_m", [None, 16, 128])
def test_mxfp8_output_ragged_then_mxfp8_input(block_m, device):
    """FC1 (SwiGLU, MXFP8 output, expert-sorted rows) feeding FC2 as MXFP8 activations (scattered, gate weights)."""
    torch.manual_seed(1)
    E, K, N = 7, 320, 448
    sizes = torch.tensor([3, 0, 1, 16, 5, 140, 2], dtype=torch.int32)
    M = int(sizes.sum())
    x = torch.randn(M, K).to(torch.bfloat16)
    w1 = torch.randn(E, K, N) * 0.05
    w2 = torch.randn(E, N // 2, 256) * 0.05
    b1, b2 = torch.randn(E, N), torch.randn(E, 256)
    v1, s1, rv1, rs1 = quantize_w(w1, device)
    v2, s2, rv2, rs2 = quantize_w(w2, device)
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    scatter = torch.randperm(M, dtype=torch.int32)
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    h_scale = torch.zeros((M, N // 2 // 32), dtype=torch.uint8, device=device)
    pc1 = PrecisionConfig(b_mx_scale=s1, b_microblock_size=32, out_dtype=torch.float8_e4m3fn, c_mx_scale=h_scale)
    with scoped_opt_flags_constraints({} if block_m is None else {"block_m": block_m}):
        h = matmul(x.to(device), v1, b1.to(device), md, precision_config=pc1, fused_activation=swiglu_act(1.702, 7.0),
                   epilogue=mxfp8_epilogue())
        h32 = matmul(x.to(device), v1, b1.to(device), md, fused_activation=swiglu_act(1.702, 7.0),
                     precision_config=PrecisionConfig(b_mx_scale=s1, b_microblock_size=32, out_dtype=torch.float32))
        want_v, want_s = downcast_to_mxfp_ref(h32.cpu(), torch.float8_e4m3fn, axis=-1)
        assert torch.equal(h_scale.cpu(), want_s) and torch.equal(h.cpu().view(torch.uint8), want_v.contiguous().view(torch.uint8))
        pc2 = PrecisionConfig(a_mx_scale=h_scale, a_microblock_size=32, b_mx_scale=s2, b_microblock_size=32)
        y = matmul(h, v2, b2.to(device), md, scatter_indx=scatter.to(device), precision_config=pc2, gammas=gammas.to(device))
    ref = MR.matmul_ref(want_v.contiguous(), rv2, b2, slice_sizes=sizes, scatter_indx=scatter, a_mx_scale=want_s,
                        b_mx_scale=rs2, gammas=gammas)
    check(y, ref)


@pytest.mark.parametrize("K", [64, 1024, 2880, 4096])
@pytest.mark.parametrize("mx", [False, True, "e5m2"])
@pytest.mark.parametrize("act", [False, True])
def test_decode_row_blocks_of_16_fp8_rows(K, mx, act, device):
    """The streaming kernel with fp8 rows (e4m3 with a per-tensor flex scale or MXFP8 block scales; e5m2 with a flex scale), expanded to bf16
    as a row block is loaded; gather, scatter with dropped rows, gate weights."""
    torch.manual_seed(K)
    E, N = 7, 608
    sizes = torch.tensor([3, 0, 1, 16, 5, 21, 2], dtype=torch.int32)
    M = int(sizes.sum())
    x0 = torch.randn(M + 5, K) * torch.exp(torch.randn(M + 5, K // 32).repeat_interleave(32, dim=1))
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s, rv, rs = quantize_w(w, device)
    gather = torch.randint(0, M + 5, (M, ), dtype=torch.int32)
    scatter = torch.randperm(M, dtype=torch.int32)
    scatter[::7] = -1
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    kw = dict(slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=rs, gammas=gammas,
              fused_swiglu=(1.702, 7.0) if act else None)
    if mx is True:
        xq, xs, rq, rxs = quantize_x_mxfp8(x0, device)
        pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32)
        ref = MR.matmul_ref(rq, rv, bias, a_mx_scale=rxs, **kw)
    else:
        fp8 = torch.float8_e5m2 if mx == "e5m2" else torch.float8_e4m3fn
        x8, x_scale = to_fp8(x0, fp8)
        xq = x8.to(device)
        pc = fp8_pc(s, x_scale, device, torch.bfloat16, fp8)
        ref = MR.matmul_ref(x8, rv, bias, a_flex_scale=x_scale, **kw).to(torch.bfloat16)
    out_init = torch.zeros((M, N // 2 if act else N), dtype=torch.bfloat16, device=device)
    with scoped_opt_flags_constraints({"block_m": 16}):
        out = matmul(xq, v, bias.to(device), md, gather_indx=gather.to(device), scatter_indx=scatter.to(device),
                     precision_config=pc, gammas=gammas.to(device), fused_activation=swiglu_act(1.702, 7.0) if act else None,
                     c=out_init)
    check(out, ref)


# ---- split-K: K cut into ranges, one launch per range into float32 partial results, summed by `reduce`, activation
# after the sum (matmul.py:180-183, 471-472, 711-737 of the reference; constraint name as in its opt_flags.py)
@pytest.mark.parametrize("M,K,N", [(64, 2048, 512), (16, 256, 64), (33, 416, 200), (130, 2880, 520)])
@pytest.mark.parametrize("split_k", [2, 3, 8])
@pytest.mark.parametrize("act", [False, True])
def test_split_k_dense(M, K, N, split_k, act, device):
    torch.manual_seed(0)
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(K, N) * 0.02
    bias = torch.randn(N)
    v, s, rv, rs = quantize_w(w, device)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    fa = swiglu_act(1.702, 7.0) if act else None
    with scoped_opt_flags_constraints({"split_k": split_k}):
        out = matmul(x.to(device), v, bias.to(device), precision_config=pc, fused_activation=fa, out_alpha=0.5)
    ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs, out_alpha=0.5, fused_swiglu=(1.702, 7.0) if act else None)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N // 2 if act else N)
    check(out, ref)


@pytest.mark.parametrize("kind", ["bf16_mxfp4", "fp8_mxfp4", "mxfp8_mxfp4", "bf16_bf16"])
def test_split_k_ragged(kind, device):
    """Gathered rows, per-row gate weights and a bias per expert: the bias must enter once, the gate weights in
    every range."""
    torch.manual_seed(1)
    E, K, N = 5, 1024, 264
    sizes = torch.tensor([7, 0, 40, 16, 130], dtype=torch.int32)
    M = int(sizes.sum())
    x0 = torch.randn(M + 3, K)
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    gather = torch.randint(0, M + 3, (M, ), dtype=torch.int32)
    gammas = 2.0**torch.randint(-3, 1, (M, )).float()
    md = make_ragged_tensor_metadata(sizes.to(device), M)
    kw = dict(slice_sizes=sizes, gather_indx=gather, gammas=gammas)
    if kind == "bf16_bf16":
        wq = w.to(torch.bfloat16)
        xq = x0.to(torch.bfloat16)
        pc, wdev = PrecisionConfig(), wq.to(device)
        ref = MR.matmul_ref(xq, wq, bias, **kw)
        xdev = xq.to(device)
    else:
        v, s, rv, rs = quantize_w(w, device)
        wdev = v
        if kind == "bf16_mxfp4":
            xq = x0.to(torch.bfloat16)
            xdev = xq.to(device)
            pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
            ref = MR.matmul_ref(xq, rv, bias, b_mx_scale=rs, **kw)
        elif kind == "fp8_mxfp4":
            x8, x_scale = to_fp8(x0)
            xdev = x8.to(device)
            pc = fp8_pc(s, x_scale, device, torch.bfloat16)
            ref = MR.matmul_ref(x8, rv, bias, a_flex_scale=x_scale, b_mx_scale=rs, **kw).to(torch.bfloat16)
        else:
            xdev, xs, rq, rxs = quantize_x_mxfp8(x0, device)
            pc = PrecisionConfig(a_mx_scale=xs, a_microblock_size=32, b_mx_scale=s, b_microblock_size=32)
            ref = MR.matmul_ref(rq, rv, bias, a_mx_scale=rxs, b_mx_scale=rs, **kw)
    with scoped_opt_flags_constraints({"split_k": 4}):
        out = matmul(xdev, wdev, bias.to(device), md, gather_indx=gather.to(device), precision_config=pc,
                     gammas=gammas.to(device))
    check(out, ref)


def test_split_k_refuses_what_it_cannot_do(device):
    from triton_amd.matmul import InapplicableConstraint
    torch.manual_seed(0)
    x = torch.randn(32, 256).to(torch.bfloat16).to(device)
    v, s, _, _ = quantize_w(torch.randn(1, 256, 64) * 0.02, device)
    md = make_ragged_tensor_metadata(torch.tensor([32], dtype=torch.int32, device=device), 32)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    scatter = torch.arange(32, dtype=torch.int32, device=device)
    with scoped_opt_flags_constraints({"split_k": 2}):
        with pytest.raises(InapplicableConstraint):
            matmul(x, v, None, md, scatter_indx=scatter, precision_config=pc)


@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.bfloat16])
@pytest.mark.parametrize("act", [False, True])
def test_split_k_with_flexpoint_output(out_dtype, act, device):
    """The ranges' float32 partial sums are finished by ONE reduction launch that applies the fused activation and the
    output's flexpoint scales (matmul.py:711-737 of the reference): same numbers as the unsplit kernel's epilogue."""
    from triton_amd.matmul import FlexCtx, OutFlexData
    torch.manual_seed(5)
    M, K, N = 48, 1024, 256
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(K, N) * 0.02
    bias = torch.randn(N)
    v, s, rv, rs = quantize_w(w, device)
    fa = swiglu_act(1.702, 7.0) if act else None
    expected = torch.tensor([0.05])
    outs = []
    for split in (1, 4):
        actual = torch.zeros(1, device=device)
        pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32, out_dtype=out_dtype, flexpoint_saturate_inf=True,
                             flex_ctx=FlexCtx(out_data=OutFlexData(expected_scale=expected.to(device), actual_scale=actual)))
        with scoped_opt_flags_constraints({"split_k": split} if split > 1 else {}):
            y = matmul(x.to(device), v, bias.to(device), precision_config=pc, fused_activation=fa)
        outs.append((y.cpu().float(), actual.cpu()))
    (y1, a1), (y4, a4) = outs
    torch.testing.assert_close(a4, a1, rtol=1e-3, atol=0)
    # fp8 outputs: one step of the type (1/8 relative) where the two summation orders round apart
    tol = dict(rtol=0.13, atol=0.5) if out_dtype == torch.float8_e4m3fn else dict(rtol=2e-2, atol=2e-1)
    torch.testing.assert_close(y4, y1, **tol)
    ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs, fused_swiglu=(1.702, 7.0) if act else None).float() / 0.05
    ref = ref.clamp(-448.0, 448.0) if out_dtype == torch.float8_e4m3fn else ref
    torch.testing.assert_close(y4, ref.to(out_dtype).float(), **tol)


@pytest.mark.parametrize("kind", ["mxfp4", "bf16"])
def test_long_k_with_few_rows_splits_by_itself(kind, device):
    """No constraint given: a dense problem with few rows and K >= 8192 is split without being asked."""
    torch.manual_seed(2)
    M, K, N = 16, 8192, 256
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(K, N) * 0.02
    bias = torch.randn(N)
    if kind == "mxfp4":
        v, s, rv, rs = quantize_w(w, device)
        out = matmul(x.to(device), v, bias.to(device), precision_config=PrecisionConfig(b_mx_scale=s, b_microblock_size=32))
        ref = MR.matmul_ref(x, rv, bias, b_mx_scale=rs)
    else:
        wq = w.to(torch.bfloat16)
        out = matmul(x.to(device), wq.to(device), bias.to(device))
        ref = MR.matmul_ref(x, wq, bias)
    check(out, ref)


@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("ragged", [False, True])
def test_mxfp8_weights(fp8, ragged, device):
    """bfloat16 x MXFP8 weights (tests/test_matmul.py:177-178 of the reference): the weights are dequantised to
    bfloat16 by the upcast kernel and multiplied by the kernel for unquantised weights."""
    from oracle.mxfp_ref import downcast_to_mxfp_ref as dref
    torch.manual_seed(3)
    E, K, N = (4, 320, 264) if ragged else (1, 416, 200)
    sizes = torch.tensor([40, 0, 130, 9], dtype=torch.int32)
    M = int(sizes.sum()) if ragged else 70
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(E, K, N) * 0.05
    bias = torch.randn(E, N)
    v, s = downcast_to_mxfp(w.to(device), fp8, axis=-2)
    rv, rs = dref(w, fp8, axis=-2)
    assert torch.equal(v.cpu().view(torch.uint8), rv.view(torch.uint8)) and torch.equal(s.cpu(), rs)
    pc = PrecisionConfig(b_mx_scale=s, b_microblock_size=32)
    if ragged:
        md = make_ragged_tensor_metadata(sizes.to(device), M)
        out = matmul(x.to(device), v, bias.to(device), md, precision_config=pc)
        ref = MR.matmul_ref(x, rv, bias, slice_sizes=sizes, b_mx_scale=rs)
    else:
        pc = PrecisionConfig(b_mx_scale=s[0], b_microblock_size=32)
        out = matmul(x.to(device), v[0], bias[0].to(device), precision_config=pc)
        ref = MR.matmul_ref(x, rv[0], bias[0], b_mx_scale=rs[0])
    check(out, ref)


@pytest.mark.parametrize("fp8", [torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("mode", ["plain", "ragged", "batched"])
def test_fp8_activations_times_fp8_weights(fp8, mode, device):
    """float8 x float8 with per-tensor flex scales on both operands (tests/test_matmul.py:150-154 of the reference),
    float32 output against the oracle, and the same problem with an fp8 flexpoint output against the cast of that."""
    from triton_amd.matmul import OutFlexData
    torch.manual_seed(4)
    E, K, N = (3, 320, 264)
    sizes = torch.tensor([40, 0, 130], dtype=torch.int32)
    M = int(sizes.sum()) if mode == "ragged" else 70
    lead = {"plain": (), "ragged": (), "batched": (E, )}[mode]
    x0 = torch.randn(*lead, M, K)
    w0 = torch.randn(*(lead if mode != "ragged" else (E, )), K, N) * 0.05
    bias = torch.randn(*(lead if mode != "ragged" else (E, )), N)
    x_scale, w_scale = (x0.abs().max() / 400).reshape(1), (w0.abs().max() / 400).reshape(1)
    x8, w8 = (x0 / x_scale).to(fp8), (w0 / w_scale).to(fp8)
    flex = FlexCtx(lhs_data=InFlexData(dtype=fp8, scale=x_scale.to(device)), rhs_data=InFlexData(dtype=fp8, scale=w_scale.to(device)))
    md = make_ragged_tensor_metadata(sizes.to(device), M) if mode == "ragged" else None
    out = matmul(x8.to(device), w8.to(device), bias.to(device), md,
                 precision_config=PrecisionConfig(flex_ctx=flex, out_dtype=torch.float32))
    ref = MR.matmul_ref(x8, w8, bias, slice_sizes=sizes if mode == "ragged" else None, a_flex_scale=x_scale,
                        b_flex_scale=w_scale)
    check(out, ref)
    expected = torch.tensor([0.25], device=device)
    actual = torch.zeros(1, device=device)
    flex8 = FlexCtx(lhs_data=flex.lhs_data, rhs_data=flex.rhs_data, out_data=OutFlexData(fp8, expected, actual, None))
    out8 = matmul(x8.to(device), w8.to(device), bias.to(device), md,
                  precision_config=PrecisionConfig(flex_ctx=flex8, flexpoint_saturate_inf=True))
    assert out8.dtype == fp8  # the output type defaults to the activations' type
    max_q = torch.finfo(fp8).max
    assert torch.equal(out8.cpu().view(torch.uint8), (out.cpu() / 0.25).clamp(-max_q, max_q).to(fp8).view(torch.uint8))
    assert actual.item() == pytest.approx(float(out.abs().max()) / max_q, rel=1e-6)
