"""GPU: the whole MoE block (routing -> up projection with SwiGLU -> down projection with gate weights and scatter
-> top-k combine) recorded into a HIP graph and replayed with new inputs.  The reference records its block the same
way (tests/test_distributed.py:311-320).  Every replay must equal the eager run on the same inputs bit for bit (same
kernels, same order of additions), and the eager run is checked against the oracle."""
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


@pytest.mark.parametrize("T", [24, 192])  # 24 tokens: row blocks of 16 (streaming kernel); 192: tiled kernel
def test_moe_block_in_a_graph(T, device):
    torch.manual_seed(0)
    E, k, H, I = 8, 2, 256, 512
    w1 = torch.randn(E, H, 2 * I) * 0.05
    w2 = torch.randn(E, I, H) * 0.05
    b1, b2 = (torch.randn(E, 2 * I) * 0.1).to(device), (torch.randn(E, H) * 0.1).to(device)
    v1, s1 = downcast_to_mxfp(w1.to(device), torch.uint8, axis=-2)
    v2, s2 = downcast_to_mxfp(w2.to(device), torch.uint8, axis=-2)
    act = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))
    logits = torch.empty(T, E, device=device)
    x = torch.empty(T, H, dtype=torch.bfloat16, device=device)

    def block():
        r = routing(logits, k)
        h = matmul(x, v1, b1, r.ragged_metadata, gather_indx=r.gather_indx,
                   precision_config=PrecisionConfig(b_mx_scale=s1, b_microblock_size=32), fused_activation=act)
        y = matmul(h, v2, b2, r.ragged_metadata, scatter_indx=r.scatter_indx,
                   precision_config=PrecisionConfig(b_mx_scale=s2, b_microblock_size=32),
                   gammas=r.expert_sorted_gate_weights)
        z, _ = reduce(y.view(T, k, H), dim=1)
        return z

    def new_inputs(seed):
        g = torch.Generator().manual_seed(seed)
        logits.copy_(torch.randn(T, E, generator=g))
        x.copy_(torch.randn(T, H, generator=g).to(torch.bfloat16))

    new_inputs(1)
    eager = block().clone()
    # the eager run against the oracle
    rr = RR.routing_ref(logits.cpu(), k)
    rv1, rs1 = downcast_to_mxfp_ref(w1, torch.uint8, axis=-2)
    rv2, rs2 = downcast_to_mxfp_ref(w2, torch.uint8, axis=-2)
    h_ref = MR.matmul_ref(x.cpu(), rv1, b1.cpu(), slice_sizes=rr["col_sum"], gather_indx=rr["gather_indx"], b_mx_scale=rs1,
                          fused_swiglu=(1.702, 7.0))
    y_ref = MR.matmul_ref(h_ref, rv2, b2.cpu(), slice_sizes=rr["col_sum"], scatter_indx=rr["scatter_indx"], b_mx_scale=rs2,
                          gammas=rr["vals"].flatten()[rr["col_sorted_indx"].long()])
    z_ref = MR.reduce_ref(y_ref.view(T, k, H), 1)
    torch.testing.assert_close(eager.cpu().float(), z_ref.float(), rtol=2e-2, atol=2e-2)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        block()  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph, stream=side):
        z_static = block()
    for seed in (1, 2, 3, 2):
        new_inputs(seed)
        graph.replay()
        replayed = z_static.clone()
        torch.cuda.synchronize()
        want = block()  # eager work between the replays, on the same inputs
        assert torch.equal(replayed, want), f"replay with inputs {seed} differs from the eager run"
    new_inputs(1)
    graph.replay()
    assert torch.equal(z_static, eager)
