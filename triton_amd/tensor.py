"""Tensor / Storage / SparseMatrix data model (tensor.py of the reference): a
torch storage plus the logical dtype and shape, which differ from the storage's
for packed FP4 data and for the bit matrix."""
from dataclasses import dataclass
from typing import Optional

import torch

from .tensor_details import bitmatrix as _bitmatrix
from .tensor_details import ragged_tensor as _ragged
from .tensor_details.dtype import (BF16, BIT, FP4, FP8_E4M3FN, FP8_E4M3FNUZ, FP8_E5M2, FP16, FP32, FP64, INT16,
                                   INT32, INT64, UINT8, DataType, FloatType, IntegerType)
from .tensor_details.layout import CDNA4MXScaleLayout, CDNA4MXValueLayout, Layout, StridedLayout
from .tensor_details.ragged_tensor import RaggedTensorMetadata
from .tensor_details.bitmatrix import BitmatrixMetadata

__all__ = ["Storage", "Tensor", "SparseMatrix", "RaggedTensorMetadata", "BitmatrixMetadata", "wrap_torch_tensor",
           "convert_layout", "empty", "make_ragged_tensor_metadata", "make_bitmatrix_metadata",
           "dtype_to_torch_dtype", "torch_dtype_to_dtype", "FP4", "UINT8", "BIT"]


@dataclass
class Storage:
    data: torch.Tensor
    layout: Layout

    @property
    def device(self):
        return self.data.device


@dataclass
class Tensor:
    storage: Storage
    dtype: DataType
    shape: Optional[list] = None
    shape_max: Optional[list] = None

    def __post_init__(self):
        assert isinstance(self.storage, Storage)
        if self.shape is None:
            if self.dtype.bitwidth < 8:
                raise ValueError("shape must be provided for sub-byte types")
            self.shape = list(self.storage.data.shape)
        self.shape = list(self.shape)
        if self.shape_max is None:
            self.shape_max = [None] * len(self.shape)
        self.shape_max = [s if m is None else m for s, m in zip(self.shape, self.shape_max)]
        for m in self.shape_max:
            if not isinstance(m, int):
                raise ValueError(f"shape_max entries must be int, got {type(m)}")

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def device(self):
        return self.storage.device

    @property
    def data(self):
        return self.storage.data

    def stride(self, i=None):
        return self.storage.data.stride() if i is None else self.storage.data.stride(i)

    def data_ptr(self):
        return self.storage.data.data_ptr()

    def numel(self):
        return self.storage.data.numel()

    def element_size(self):
        return self.dtype.bitwidth // 8

    def dim(self):
        return self.ndim

    def size(self, i=None):
        return self.shape if i is None else self.shape[i]


_TO_TORCH = {
    FP4: torch.uint8, UINT8: torch.uint8, FP8_E4M3FN: torch.float8_e4m3fn, FP8_E4M3FNUZ: torch.float8_e4m3fnuz,
    FP8_E5M2: torch.float8_e5m2, BF16: torch.bfloat16, FP16: torch.float16, FP32: torch.float32,
    FP64: torch.float64, INT16: torch.int16, INT32: torch.int32, INT64: torch.int64,
}
_FROM_TORCH = {
    torch.uint8: UINT8, torch.float8_e4m3fn: FP8_E4M3FN, torch.float8_e4m3fnuz: FP8_E4M3FNUZ,
    torch.float8_e5m2: FP8_E5M2, torch.float16: FP16, torch.bfloat16: BF16, torch.float32: FP32,
    torch.float64: FP64, torch.int16: INT16, torch.int32: INT32, torch.int64: INT64,
}


def dtype_to_torch_dtype(dtype):
    if dtype is None or isinstance(dtype, torch.dtype):
        return dtype
    return _TO_TORCH[dtype]


def torch_dtype_to_dtype(dtype):
    if isinstance(dtype, (IntegerType, FloatType)):
        return dtype
    if dtype in _FROM_TORCH:
        return _FROM_TORCH[dtype]
    raise AssertionError(f"Unknown dtype: {dtype}")


def wrap_torch_tensor(torch_tensor: torch.Tensor, dtype=None, shape=None, shape_max=None, layout=None) -> Tensor:
    """Wraps a torch tensor.  For FP4 the logical shape doubles the unit-stride axis
    (two codes per byte); the layout records which axis that is."""
    t = torch_tensor
    dtype = torch_dtype_to_dtype(t.dtype if dtype is None else dtype)
    strides = list(t.stride())
    if shape is None:
        shape = list(t.shape)
        if dtype == FP4:
            shape[strides.index(1)] *= (8 * t.dtype.itemsize) // dtype.bitwidth
    if shape_max is None:
        shape_max = list(shape)
    if layout is None:
        major = strides.index(1) if 1 in strides else t.ndim - 1
        layout = StridedLayout(major_dim=major - t.ndim)
    return Tensor(Storage(t, layout), dtype=dtype, shape=shape, shape_max=shape_max)


def empty(shape, dtype, device, layout=None, allow_implicit_conversion: bool = False) -> Tensor:
    """Uninitialised tensor whose storage is contiguous along layout.major_dim (reference tensor.py:300-317).  A
    layout that is not strided is only accepted with `allow_implicit_conversion`: the tensor is then allocated in
    the default strided layout and converted."""
    initial = layout if isinstance(layout, StridedLayout) else StridedLayout()
    is_fp4 = dtype == FP4
    sshape = initial.storage_shape(list(shape), is_fp4)
    data = torch.empty_strided(sshape, initial.strides(sshape), dtype=dtype_to_torch_dtype(dtype), device=device)
    ret = Tensor(Storage(data, initial), dtype=dtype, shape=list(shape))
    assert layout is None or initial == layout or allow_implicit_conversion
    if allow_implicit_conversion and layout is not None and initial != layout:
        ret = convert_layout(ret, layout)
    return ret


def convert_layout(tensor: Tensor, layout: Layout) -> Tensor:
    """Re-encodes `tensor` in `layout`: another contiguous (packed) axis, or the CDNA4 scale pre-shuffle and back
    (reference tensor.py:235-252).  Returns `tensor` itself when its storage already has that encoding."""
    src = tensor.storage.layout
    if isinstance(src, CDNA4MXValueLayout) or isinstance(layout, CDNA4MXValueLayout):
        if src == layout:
            return tensor
        assert tensor.dtype == FP4, "the CDNA4 value layout holds packed e2m1 codes"
        if isinstance(src, CDNA4MXValueLayout):
            data = src.make_transformation(tensor.shape).unswizzle_data(tensor.storage.data)   # unit stride along K
            strided = Tensor(Storage(data, StridedLayout(-2)), dtype=FP4, shape=list(tensor.shape))
            return convert_layout(strided, layout)
        k_major = convert_layout(tensor, StridedLayout(-2))   # packed along K, whatever the source packs along
        data = layout.make_transformation(tensor.shape).swizzle_data(k_major.storage.data)
        return Tensor(Storage(data, layout), dtype=FP4, shape=list(tensor.shape))
    if isinstance(src, CDNA4MXScaleLayout) or isinstance(layout, CDNA4MXScaleLayout):
        if src == layout:
            return tensor
        assert tensor.dtype != FP4, "the CDNA4 scale layout holds bytes"
        data = tensor.storage.data
        if isinstance(src, CDNA4MXScaleLayout):
            data = src.make_transformation(tensor.shape).unswizzle_data(data)
        if isinstance(layout, CDNA4MXScaleLayout):
            data = layout.make_transformation(tensor.shape).swizzle_data(data)
            return Tensor(Storage(data, layout), dtype=tensor.dtype, shape=list(tensor.shape))
        return convert_layout(wrap_torch_tensor(data, dtype=tensor.dtype), layout)
    if not isinstance(layout, StridedLayout) or not isinstance(src, StridedLayout):
        raise NotImplementedError(f"layout {type(layout).__name__} does not exist on gfx950")
    rank = tensor.ndim
    if tensor.storage.layout.order(rank) == layout.order(rank):
        return tensor
    if tensor.dtype == FP4:
        src_axis = tensor.storage.layout.order(rank)[0]
        dst_axis = layout.order(rank)[0]
        data = tensor.storage.data
        lo, hi = data & 0xF, data >> 4
        codes = torch.stack([lo, hi], dim=src_axis + 1).flatten(src_axis, src_axis + 1)  # one code per byte
        codes = codes.movedim(dst_axis, -1)
        packed = (codes[..., 0::2] | (codes[..., 1::2] << 4)).movedim(-1, dst_axis)
        out = empty(tensor.shape, FP4, data.device, layout)
        out.storage.data.copy_(packed)
        return out
    out = empty(tensor.shape, tensor.dtype, tensor.device, layout)
    out.storage.data.copy_(tensor.storage.data)
    return out


make_ragged_tensor_metadata = _ragged.make_ragged_tensor_metadata
make_bitmatrix_metadata = _bitmatrix.make_bitmatrix_metadata


@dataclass
class SparseMatrix:
    """Top-k result: `indx`/`vals` [n_rows, k], `mask` the bit matrix; building one
    computes the histogram / ordering metadata, as in the reference (tensor.py:203-210)."""
    indx: torch.Tensor
    vals: torch.Tensor
    mask: Tensor

    def __post_init__(self):
        self.mask_metadata = make_bitmatrix_metadata(self.indx, self.mask)
