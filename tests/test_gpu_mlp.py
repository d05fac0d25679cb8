"""GPU parity of the whole MoE layer as the reference's bench/bench_mlp.py:60-96 chains it on one rank:
gate matmul -> top-k + softmax -> metadata -> FC1 + SwiGLU (gathered rows) -> FC2 (rows scattered back) -> sum over k.
Every stage is checked against the oracle fed with the GPU's output of the stage before (integers bit-exact), and the
end of the chain against an oracle chain that only shares the gate logits."""
import pytest
import torch

from oracle import matmul_ref as MR
from oracle import routing_ref as RR
from oracle.mxfp_ref import downcast_to_mxfp_ref
from triton_amd.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
from triton_amd.numerics_details.mxfp import downcast_to_mxfp
from triton_amd.reduce import reduce
from triton_amd.routing import routing
from triton_amd.swiglu import swiglu_fn

pytestmark = pytest.mark.gpu


def _quantise(w, device):
    """[E, K, N] float32 -> MXFP4 along K on the GPU (what the matmul consumes) and by the oracle (what it is checked with)."""
    v, s = downcast_to_mxfp(w.to(torch.bfloat16).to(device), torch.uint8, axis=1)
    rv, rs = downcast_to_mxfp_ref(w.to(torch.bfloat16), torch.uint8, 1)
    assert torch.equal(v.cpu(), rv) and torch.equal(s.cpu(), rs)
    return v, s, rv, rs


@pytest.mark.parametrize("T,E,k,d1,d2,x_dtype", [(200, 16, 4, 768, 768, torch.float8_e4m3fn), (64, 32, 4, 512, 1024, torch.float8_e4m3fn),
                                                 (333, 8, 2, 768, 512, torch.bfloat16)])
def test_mlp_layer(T, E, k, d1, d2, x_dtype, device):
    torch.manual_seed(0)
    wg = torch.randn(d1, E).to(torch.bfloat16)
    bg, b1, b2 = torch.randn(E), torch.randn(E, d2), torch.randn(E, d1)
    w1, s1, rw1, rs1 = _quantise(torch.randn(E, d1, d2), device)
    w2, s2, rw2, rs2 = _quantise(torch.randn(E, d2 // 2, d1), device)
    x = torch.randn(T, d1).to(x_dtype)
    x16 = x.to(torch.bfloat16)
    pc1 = PrecisionConfig(b_mx_scale=s1, b_microblock_size=32)
    pc2 = PrecisionConfig(b_mx_scale=s2, b_microblock_size=32)
    act1 = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.0, 1.0))
    # ---- the layer on the GPU
    wg_dev = wg.to(device).t().contiguous().t()  # unit stride along K, as the reference's quantize_weight leaves bf16 weights
    logits = matmul(x16.to(device), wg_dev, bg.to(device))
    r = routing(logits, k)
    y1 = matmul(x.to(device), w1, b1.to(device), r.ragged_metadata, gather_indx=r.gather_indx, precision_config=pc1,
                fused_activation=act1)
    y2 = matmul(y1, w2, b2.to(device), r.ragged_metadata, scatter_indx=r.scatter_indx, precision_config=pc2)
    z, _ = reduce(y2.view(T, k, d1), dim=1)
    assert y1.dtype == x_dtype and y2.dtype == x_dtype and z.dtype == x_dtype and tuple(z.shape) == (T, d1)
    # ---- stage by stage
    fp8 = x_dtype == torch.float8_e4m3fn
    tol = dict(rtol=0.13, atol=2e-2) if fp8 else dict(rtol=2e-2, atol=2e-2)  # one step of the output type
    logits_ref = MR.matmul_ref(x16, wg, bg)
    torch.testing.assert_close(logits.cpu().float(), logits_ref.float(), rtol=2e-2, atol=2e-1)
    ref = RR.routing_ref(logits.cpu(), k)
    assert torch.equal(r.indx.cpu().int(), ref["indx"]) and torch.equal(r.col_sum.cpu(), ref["col_sum"])
    assert torch.equal(r.gather_indx.cpu(), ref["gather_indx"]) and torch.equal(r.scatter_indx.cpu(), ref["scatter_indx"])
    y1_ref = MR.matmul_ref(x, rw1, b1, slice_sizes=ref["col_sum"], gather_indx=ref["gather_indx"], b_mx_scale=rs1,
                           fused_swiglu=(1.0, 1.0))
    torch.testing.assert_close(y1.cpu().float(), y1_ref.float(), **tol)
    y2_ref = MR.matmul_ref(y1.cpu(), rw2, b2, slice_sizes=ref["col_sum"], scatter_indx=ref["scatter_indx"], b_mx_scale=rs2)
    a, b = y2.cpu().float(), y2_ref.float()
    assert torch.equal(torch.isnan(a), torch.isnan(b)) or fp8  # fp8 sums at the overflow boundary may differ by a step
    torch.testing.assert_close(torch.nan_to_num(a, nan=0.0), torch.nan_to_num(b, nan=0.0), rtol=tol["rtol"], atol=1.0 if fp8 else 0.5)
    z_ref, _, _ = MR.reduce_general_ref(y2.view(T, k, d1).cpu(), 1)
    zc, zr = z.cpu().float(), z_ref.float()
    assert torch.equal(torch.isnan(zc), torch.isnan(zr)) and torch.equal(torch.nan_to_num(zc), torch.nan_to_num(zr))
    # ---- the end of the chain against an oracle chain that shares only the routing decision
    y2_chain = MR.matmul_ref(y1_ref, rw2, b2, slice_sizes=ref["col_sum"], scatter_indx=ref["scatter_indx"], b_mx_scale=rs2)
    z_chain, _, _ = MR.reduce_general_ref(y2_chain.view(T, k, d1), 1)
    good = torch.isfinite(zc) & torch.isfinite(z_chain.float())
    assert good.float().mean() > 0.99
    err = (zc[good] - z_chain.float()[good]).norm() / z_chain.float()[good].norm()
    assert err < (0.08 if fp8 else 0.02), f"relative error of the layer output {err:.3f}"
