"""The vectors of tests/golden/reference_vectors.json (what the reference's tests and docstrings spell out) against
the CPU oracle, and against the HIP path through the C ABI (GPU-marked tests)."""
import json
import os

import pytest
import torch

from oracle import mxfp_ref as MX
from oracle import routing_ref as RR

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}


def _rounding_input(name):
    g = G["mxfp4_rounding"]
    vals = g["x_head"] + [g["x_tie_plus_one_ulp"][name]]
    return torch.tensor(vals + [0] * (g["axis_len"] - len(vals)), dtype=DTYPES[name]).view(1, -1)


def _check_rounding(name, down, up):
    g = G["mxfp4_rounding"]
    q, s = down(_rounding_input(name))
    assert s.flatten().tolist() == [g["scale_byte"]]
    assert q.flatten().tolist()[:5] == g["packed_head"]
    d = up(q, s, DTYPES[name])
    assert d.flatten().tolist() == g["dequantised_head"] + [0] * (g["axis_len"] - len(g["dequantised_head"]))


def _check_round_down(down, up, rounding):
    g = G["mxfp4_round_down"]
    x = torch.tensor(g["x"] + [0] * 24).bfloat16().view(1, -1)
    q, s = down(x, rounding)
    assert s.item() == g["scale_byte"]
    assert up(q, s, torch.float32).flatten().tolist()[:8] == g["dequantised"]


def _check_upcast_247(up):
    g = G["mxfp4_upcast_scale_247"]
    q = torch.tensor([g["packed"] + [0] * 15], dtype=torch.uint8)
    s = torch.tensor([[g["scale_byte"]]], dtype=torch.uint8)
    d = up(q, s, torch.float32)
    assert [d[0, 0].item() / 2.0**120, d[0, 1].item() / 2.0**120] == g["values_times_2_pow_minus_120"]


@pytest.mark.parametrize("name", list(DTYPES))
def test_oracle_mxfp_vectors(name):
    _check_rounding(name, lambda x: MX.downcast_to_mxfp_ref(x, torch.uint8, axis=1),
                    lambda q, s, dt: MX.upcast_from_mxfp_ref(q, s, dt, axis=1))
    _check_round_down(lambda x, r: MX.downcast_to_mxfp_ref(x, torch.uint8, axis=1, rounding=r),
                      lambda q, s, dt: MX.upcast_from_mxfp_ref(q, s, dt, axis=1), "down")
    _check_upcast_247(lambda q, s, dt: MX.upcast_from_mxfp_ref(q, s, dt, axis=1))
    codes = torch.arange(16, dtype=torch.uint8)
    packed = (codes[0::2] | (codes[1::2] << 4)).view(1, -1)  # one byte = two codes, 16 values; pad the group with zeros
    packed = torch.cat([packed, torch.zeros(1, 8, dtype=torch.uint8)], dim=1)
    vals = MX.upcast_from_mxfp_ref(packed, torch.tensor([[127]], dtype=torch.uint8), torch.float32, axis=1)[0, :16].tolist()
    mags = G["e2m1_value_table"]["magnitudes"]
    assert vals == mags + [-m for m in mags]


def _bitmatrix_indx():
    m = G["bitmatrix_metadata"]["matrix"]
    return torch.tensor([c for row in m for c, bit in enumerate(row) if bit], dtype=torch.int32).view(-1, 1), len(m[0])


def test_oracle_routing_vectors():
    g = G["bitmatrix_metadata"]
    indx, n_cols = _bitmatrix_indx()
    m = RR.bitmatrix_metadata_ref(indx, n_cols)
    assert m.col_sum.tolist() == g["col_sum"]
    assert m.col_sorted_indx.tolist() == g["col_sorted_indx"]
    assert m.row_sorted_indx.tolist() == g["row_sorted_indx"]
    g = G["ragged_metadata"]
    r = RR.ragged_metadata_ref(torch.tensor(g["slice_sizes"], dtype=torch.int32), sum(g["slice_sizes"]))
    assert r.slice_offs.tolist() == g["slice_offs"]
    for i, b in enumerate(RR.BLOCK_SIZES):
        if str(b) in g["block_offs"]:
            assert r.block_offs_data[i].tolist() == g["block_offs"][str(b)]
    sched = [[v >> 16, v & 0xFFFF] for v in r.block_schedule_data[RR.BLOCK_SIZES.index(32)].tolist() if v != -1]
    assert sched == g["block_schedule_32"]


def test_layout_vectors():
    from oracle import layout_ref as LR
    from triton_amd.tensor_details.layout import CDNA4MXScaleLayout, StridedLayout
    for case in G["cdna4_scale_storage_shapes"]["cases"]:
        assert LR.cdna4_storage_shape(case["shape"]) == case["storage"]
        assert CDNA4MXScaleLayout().storage_shape(list(case["shape"]), False) == case["storage"]
    g = G["fp4_strided_storage_shape"]
    assert StridedLayout(g["major_dim"]).storage_shape(g["shape"], True) == g["storage"]


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(DTYPES))
def test_gpu_mxfp_vectors(name, device):
    from triton_amd.numerics_details.mxfp import DequantScaleRoundingMode, downcast_to_mxfp, upcast_from_mxfp
    cpu = lambda pair: tuple(t.cpu() for t in pair)
    up = lambda q, s, dt: upcast_from_mxfp(q.to(device), s.to(device), dt, axis=1).cpu()
    _check_rounding(name, lambda x: cpu(downcast_to_mxfp(x.to(device), torch.uint8, axis=1)), up)
    _check_round_down(lambda x, r: cpu(downcast_to_mxfp(x.to(device), torch.uint8, axis=1,
                                                        DEQUANT_SCALE_ROUNDING_MODE=DequantScaleRoundingMode.ROUND_DOWN)), up, "down")
    _check_upcast_247(up)


@pytest.mark.gpu
def test_gpu_routing_vectors(device):
    from triton_amd.tensor import BIT, make_bitmatrix_metadata, make_ragged_tensor_metadata, wrap_torch_tensor
    g = G["bitmatrix_metadata"]
    indx, n_cols = _bitmatrix_indx()
    bm = wrap_torch_tensor(torch.zeros((indx.shape[0], 1), dtype=torch.int32, device=device).view(torch.uint32), dtype=BIT,
                           shape=(indx.shape[0], n_cols))
    m = make_bitmatrix_metadata(indx.to(device), bm)
    assert m.col_sum.cpu().tolist() == g["col_sum"]
    assert m.col_sorted_indx.cpu().tolist() == g["col_sorted_indx"]
    assert m.row_sorted_indx.cpu().tolist() == g["row_sorted_indx"]
    g = G["ragged_metadata"]
    md = make_ragged_tensor_metadata(torch.tensor(g["slice_sizes"], dtype=torch.int32, device=device), sum(g["slice_sizes"]))
    assert md.slice_offs.cpu().tolist() == g["slice_offs"]
    for b, want in g["block_offs"].items():
        assert md.block_offs(int(b)).cpu().tolist()[:len(want)] == want
    sched = [[v >> 16, v & 0xFFFF] for v in md.block_schedule(32).cpu().tolist() if v != -1]
    assert sched == g["block_schedule_32"]
