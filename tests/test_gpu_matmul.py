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
from triton_amd.tensor import make_ragged_tensor_metadata
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


@pytest.mark.parametrize("M,K,N", [(256, 2048, 4096), (16, 64, 64), (33, 96, 200), (130, 192, 520), (1, 32, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dense(M, K, N, dtype, device):
    """(256, 2048, 4096) is BASELINE config 1."""
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


def to_fp8(x0):
    """Per-tensor flex quantisation as in BASELINE config 5: s = amax / 448, x = (x0 / s) -> e4m3."""
    s = x0.abs().max() / 448.0
    return (x0 / s).to(torch.float8_e4m3fn), s.reshape(1).float()


def fp8_pc(s_w, x_scale, device, out_dtype):
    flex = FlexCtx(lhs_data=InFlexData(dtype=torch.float8_e4m3fn, scale=x_scale.to(device)))
    return PrecisionConfig(b_mx_scale=s_w, b_microblock_size=32, flex_ctx=flex, out_dtype=out_dtype)


@pytest.mark.parametrize("M,K,N", [(256, 2048, 512), (16, 64, 64), (33, 96, 200), (130, 192, 520), (1, 32, 16),
                                   (128, 2880, 256)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_fp8_dense(M, K, N, out_dtype, device):
    torch.manual_seed(0)
    x8, xs = to_fp8(torch.randn(M, K))
    w = torch.randn(K, N) * 0.02
    bias = torch.randn(N) * 0.1
    v, s, rv, rs = quantize_w(w, device)
    out = matmul(x8.to(device), v, bias.to(device), precision_config=fp8_pc(s, xs, device, out_dtype))
    ref = MR.matmul_ref(x8, rv, bias, b_mx_scale=rs, a_flex_scale=xs)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    check(out, ref.to(out_dtype))


def test_fp8_one_hot_rows_are_exact(device):
    """x = one-hot rows (1.0 is exact in e4m3): the scaled MFMA must return the dequantised weight rows bit for
    bit, which pins the K order of both operands and the scale-byte selection."""
    torch.manual_seed(1)
    K, N = 256, 256
    w = torch.randn(K, N)
    v, s, rv, rs = quantize_w(w, device)
    x8 = torch.eye(K)[:160].to(torch.float8_e4m3fn)
    one = torch.ones(1)
    out = matmul(x8.to(device), v, None, precision_config=fp8_pc(s, one, device, torch.float32))
    from oracle.mxfp_ref import upcast_from_mxfp_ref
    deq = upcast_from_mxfp_ref(rv, rs, torch.float32, axis=0)
    assert torch.equal(out.cpu(), deq[:160])


@pytest.mark.parametrize("block_m", [None, 16, 32, 64, 128])
@pytest.mark.parametrize("do_gather,do_scatter,do_gamma,act", [(False, False, False, False), (True, False, False, True),
                                                                (False, True, True, False)])
def test_fp8_ragged(block_m, do_gather, do_scatter, do_gamma, act, device):
    torch.manual_seed(0)
    E, K, N, M = 9, 320, 392, 700
    sizes = torch.tensor([0, 5, 130, 16, 1, 257, 64, 200, 27], dtype=torch.int32)
    x8, xs = to_fp8(torch.randn(M, K))
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
                     precision_config=fp8_pc(s, xs, device, torch.bfloat16), gammas=dev(gammas), fused_activation=fa,
                     c=out_init)
    ref = MR.matmul_ref(x8, rv, bias, slice_sizes=sizes, gather_indx=gather, scatter_indx=scatter, b_mx_scale=rs,
                        a_flex_scale=xs, gammas=gammas, fused_swiglu=(1.702, 7.0) if act else None)
    check(out, ref.to(torch.bfloat16))


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
