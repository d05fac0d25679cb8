"""CDNA4 scale pre-shuffle: the oracle against what the reference's tests spell out, and the host implementation
against the oracle (CPU only)."""
import numpy as np
import pytest
import torch

from oracle import layout_ref as LR
from triton_amd.tensor import UINT8, convert_layout, empty, wrap_torch_tensor
from triton_amd.tensor_details.layout import (CDNA4MXScaleLayout, StridedLayout,
                                              make_default_matmul_mxfp4_w_scale_layout)

ROUNDTRIP_SHAPES = [(3, 4096, 1024), (10, 254, 60), (1, 320, 160), (2, 16, 512), (3, 2, 36)]  # test_layout_cdna4.py:26-32
ZERO_SHAPES = [(0, 64), (64, 0), (2, 0), (0, 2), (0, 64, 64)]  # test_layout_cdna4.py:11


@pytest.mark.parametrize("shape,storage", [((3, 254, 60), [3, 8192, 2]), ((0, 64), [1, 0, 2])])  # test_tensor.py:52-53
def test_storage_shape_literals(shape, storage):
    assert LR.cdna4_storage_shape(shape) == storage
    assert CDNA4MXScaleLayout().storage_shape(list(shape), False) == storage
    t = empty(shape, UINT8, "meta")
    assert list(convert_layout(t, CDNA4MXScaleLayout()).storage.data.shape) == storage


@pytest.mark.parametrize("shape", ROUNDTRIP_SHAPES)
def test_oracle_roundtrip_and_kernel_side_inverse(shape):
    rng = np.random.default_rng(0)
    x = rng.integers(0, 256, size=shape, dtype=np.uint8)
    flat = LR.cdna4_swizzle_ref(x)
    assert np.array_equal(LR.cdna4_unswizzle_ref(flat, shape), x)
    # what the reference's kernel does to a block it loaded must recover the logical block
    b, rows, blocks = LR.cdna4_storage_shape(shape)
    kp, npad = rows // 32, blocks * 32
    for bi in range(min(b, 2)):
        got = LR.cdna4_block_unswizzle_ref(flat[bi].reshape(blocks, kp * 32), npad, kp)
        want = np.zeros((npad, kp), dtype=np.uint8)
        want[:shape[-1], :shape[-2]] = x.reshape(b, shape[-2], shape[-1])[bi].T
        assert np.array_equal(got, want)


def test_oracle_small_case_by_hand():
    """One block of 32 columns x 8 groups: byte 0 is (k 0, n 0), byte 1 is (k 0, n 16), byte 2 is (k 4, n 0),
    byte 4 is (k 0, n 1), byte 64 is (k 1, n 0)."""
    x = np.arange(8 * 32, dtype=np.uint16).reshape(8, 32)  # value = 32*k + n
    flat = LR.cdna4_swizzle_ref(x)[0]
    assert [int(flat[i]) for i in (0, 1, 2, 3, 4, 64, 255)] == [0, 16, 4 * 32, 4 * 32 + 16, 1, 32, 7 * 32 + 31]


@pytest.mark.parametrize("shape", ROUNDTRIP_SHAPES + ZERO_SHAPES)
def test_host_swizzle_matches_oracle(shape):
    torch.manual_seed(0)
    x = torch.randint(0, 256, shape, dtype=torch.uint8)
    src = wrap_torch_tensor(x)
    sw = convert_layout(src, CDNA4MXScaleLayout())
    data = sw.storage.data
    assert list(data.shape) == LR.cdna4_storage_shape(shape) and sw.shape == list(shape)
    assert data.numel() == 0 or data.stride(-2) == 1
    flat = data.transpose(-1, -2).reshape(data.shape[0], data.shape[1] * data.shape[2]).numpy()
    assert np.array_equal(flat, LR.cdna4_swizzle_ref(x.numpy()))
    back = convert_layout(sw, src.storage.layout)
    assert back.storage.data.shape == x.shape and torch.equal(back.storage.data, x)
    assert convert_layout(sw, CDNA4MXScaleLayout()) is sw


def test_swizzle_of_a_k_contiguous_view():
    """Scales as downcast_to_mxfp returns them ([E, K/32, N] with unit stride along K/32)."""
    x = torch.randint(0, 256, (2, 96, 90), dtype=torch.uint8).transpose(1, 2)  # [2, 90, 96], stride (.., 1, 90)
    sw = convert_layout(wrap_torch_tensor(x), CDNA4MXScaleLayout())
    flat = sw.storage.data.transpose(-1, -2).reshape(2, -1).numpy()
    assert np.array_equal(flat, LR.cdna4_swizzle_ref(x.contiguous().numpy()))


def test_default_scale_layout_is_the_preshuffle():
    assert isinstance(make_default_matmul_mxfp4_w_scale_layout(mx_axis=1), CDNA4MXScaleLayout)
    assert CDNA4MXScaleLayout().name == "CDNA4_SCALE" and StridedLayout(-2).name == "STRIDED"
    assert CDNA4MXScaleLayout().swizzle_block_shape([4, 256]) == [8, 128]
