"""CDNA4 scale pre-shuffle: the oracle against what the reference's tests spell out, and the host implementation
against the oracle (CPU only)."""
import numpy as np
import pytest
import torch

from oracle import layout_ref as LR
from triton_amd.tensor import FP4, UINT8, convert_layout, empty, wrap_torch_tensor
from triton_amd.tensor_details.layout import (CDNA4MXScaleLayout, CDNA4MXValueLayout, StridedLayout,
                                              make_default_matmul_mxfp4_w_scale_layout, make_native_matmul_mxfp4_w_layout)

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


# ---- the MXFP4 value layout of the gfx950 kernels -------------------------------------------------------------------
VALUE_SHAPES = [(1, 128, 64), (2, 256, 192), (3, 320, 160), (1, 2880, 128), (2, 96, 36), (64, 64), (1, 130, 2)]


def test_value_layout_offsets_by_hand():
    """A block is 4 KB: 64 positions of 64 bytes; column n = 2c + f of a strip is position 32 f + c; the four 16-byte
    parts of a position are rotated by ((c >> 2) & 3) ^ 2 f; blocks follow each other along K inside a strip."""
    off = LR.cdna4_value_offset
    assert off(0, 0, 3) == 0                                  # first byte of column 0
    assert off(15, 0, 3) == 15 and off(16, 0, 3) == 16        # column 0: c = 0, f = 0, no rotation
    assert off(0, 1, 3) == 32 * 64 + 2 * 16                   # column 1: f = 1 -> position 32, slot 0 ^ 2
    assert off(0, 2, 3) == 64                                 # column 2: c = 1 -> position 1
    assert off(0, 8, 3) == 4 * 64 + 1 * 16                    # column 8: c = 4 -> rotation 1
    assert off(48, 8, 3) == 4 * 64 + (3 ^ 1) * 16             # its last part sits in slot 2
    assert off(64, 0, 3) == 4096                              # next K stage: next block of the strip
    assert off(0, 64, 3) == 3 * 4096                          # next strip: after the strip's three stages
    assert off(0, 127, 3) == 3 * 4096 + 63 * 64 + (0 ^ 3 ^ 2) * 16   # c = 31, f = 1: rotation (7 & 3) ^ 2 = 1
    assert LR.cdna4_value_storage_shape((3, 2880, 5760)) == [3, 90, 23 * 4096]
    assert LR.cdna4_value_storage_shape((130, 2)) == [1, 1, 2 * 4096]


@pytest.mark.parametrize("shape", VALUE_SHAPES)
def test_value_layout_oracle_roundtrip_and_host_match(shape):
    rng = np.random.default_rng(1)
    *lead, k, n = shape
    x = rng.integers(0, 256, size=(*lead, k // 2, n), dtype=np.uint8)
    stored = LR.cdna4_value_swizzle_ref(x)
    assert list(stored.shape) == LR.cdna4_value_storage_shape(shape)
    assert np.array_equal(LR.cdna4_value_unswizzle_ref(stored, shape), x)
    # every byte of the input appears exactly once, everything else is padding (zero)
    assert np.sort(stored[stored != 0]).tolist() == np.sort(x[x != 0]).tolist()
    # the product's torch implementation, from the layout downcast_to_mxfp produces (unit stride along K) and from a
    # row-major copy
    xt = torch.from_numpy(x)
    k_major = xt.transpose(-1, -2).contiguous().transpose(-1, -2)
    for src in (k_major, xt):
        t = wrap_torch_tensor(src, dtype=FP4, shape=list(shape), layout=StridedLayout(-2)) if src is k_major else None
        if t is None:
            continue
        sw = convert_layout(t, CDNA4MXValueLayout())
        assert sw.shape == list(shape) and list(sw.storage.data.shape) == list(stored.shape)
        assert sw.storage.data.is_contiguous() and np.array_equal(sw.storage.data.numpy(), stored)
        assert convert_layout(sw, CDNA4MXValueLayout()) is sw
        back = convert_layout(sw, StridedLayout(-2))
        assert back.shape == list(shape) and back.storage.data.stride(-2) == 1
        assert torch.equal(back.storage.data, xt)


def test_value_layout_from_codes_packed_along_n():
    """A tensor whose codes are packed along N (StridedLayout(-1)) converts through the K-packed form."""
    torch.manual_seed(2)
    codes = torch.randint(0, 16, (2, 128, 64), dtype=torch.uint8)            # one code per entry, [B, K, N]
    along_n = codes[..., 0::2] | (codes[..., 1::2] << 4)                      # [B, K, N/2]
    along_k = (codes[:, 0::2, :] | (codes[:, 1::2, :] << 4))                  # [B, K/2, N]
    t = wrap_torch_tensor(along_n, dtype=FP4, shape=[2, 128, 64], layout=StridedLayout(-1))
    sw = convert_layout(t, CDNA4MXValueLayout())
    assert np.array_equal(sw.storage.data.numpy(), LR.cdna4_value_swizzle_ref(along_k.numpy()))


def test_native_value_layout_names():
    assert isinstance(make_native_matmul_mxfp4_w_layout(mx_axis=1), CDNA4MXValueLayout)
    assert CDNA4MXValueLayout().name == "CDNA4_VALUE"
    assert CDNA4MXValueLayout().storage_shape([128, 2880, 5760]) == [128, 90, 23 * 4096]
    from triton_amd.tensor_details.layout_details import cdna4_value
    assert cdna4_value.CDNA4MXValueLayout is CDNA4MXValueLayout
