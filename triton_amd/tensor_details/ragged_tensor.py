"""Ragged tensor metadata (tensor_details/ragged_tensor.py of the reference):
slice offsets, per-block-size block offsets and the tile schedule consumed by
the grouped matmul."""
from dataclasses import dataclass
from typing import Optional

import torch

from .. import _lib

_PITCH = 512  # rows of both tables are padded to this many elements (ragged_tensor.py:106-111, 192-193)


@dataclass
class RaggedTensorMetadata:
    slice_sizes: torch.Tensor        # int32 [n_slices]
    slice_offs: torch.Tensor         # int32 [n_slices+1] = [0] + cumsum(slice_sizes)
    block_offs_data: torch.Tensor    # int32 [5, n_slices+1], block sizes 16..256
    block_schedule_data: torch.Tensor  # int32 [5, max_n_blocks], (block << 16) | slice, -1 padding
    expected_slice_size: Optional[int] = None
    slice_sizes_divisibility: Optional[int] = None

    def __post_init__(self):
        n = len(self.block_sizes())
        assert self.block_offs_data.shape[0] == n and self.block_schedule_data.shape[0] == n
        assert self.block_offs_data.dtype == torch.int32 and self.block_schedule_data.dtype == torch.int32
        assert self.slice_sizes is None or self.slice_sizes.dtype == torch.int32
        assert self.slice_offs is None or self.slice_offs.dtype == torch.int32

    @property
    def n_slices(self):
        return self.slice_sizes.shape[0]

    @staticmethod
    def block_sizes_log2():
        return range(4, 9)

    @staticmethod
    def block_sizes():
        return [1 << s for s in RaggedTensorMetadata.block_sizes_log2()]

    def block_offs(self, block_size):
        return self.block_offs_data[self.block_sizes().index(block_size)]

    def block_schedule(self, block_size):
        return self.block_schedule_data[self.block_sizes().index(block_size)]

    @staticmethod
    def n_blocks(n_slices, n_total_rows, block_size):
        """Largest possible number of row blocks for any split of the rows."""
        if n_total_rows <= n_slices:
            return n_total_rows
        return n_slices - 1 - ((n_slices - n_total_rows - 1) // block_size)

    @staticmethod
    def max_n_blocks(n_slices, n_total_rows):
        return RaggedTensorMetadata.n_blocks(n_slices, n_total_rows, min(RaggedTensorMetadata.block_sizes()))


def _padded(rows, cols, device):
    pitch = -(-max(cols, 1) // _PITCH) * _PITCH
    return torch.empty((rows, pitch), dtype=torch.int32, device=device)


def alloc_tables(n_slices, n_total_rows, device):
    width = RaggedTensorMetadata.max_n_blocks(n_slices, n_total_rows)
    offs = _padded(6, n_slices + 1, device)
    sched = _padded(5, width, device)
    return offs, sched, width


def make_ragged_tensor_metadata(slice_sizes: torch.Tensor, n_total_rows: int) -> RaggedTensorMetadata:
    assert slice_sizes.ndim == 1
    assert slice_sizes.dtype == torch.int32
    _lib.require_gpu(slice_sizes, "slice_sizes")
    slice_sizes = slice_sizes.contiguous()
    n = slice_sizes.shape[0]
    offs, sched, width = alloc_tables(n, n_total_rows, slice_sizes.device)
    rc = _lib.lib().tamd_ragged_metadata(_lib.ptr(slice_sizes), n, _lib.ptr(offs), offs.stride(0), _lib.ptr(sched),
                                         sched.stride(0), width, _lib.stream_ptr(slice_sizes.device))
    _lib.check(rc, "make_ragged_tensor_metadata")
    return RaggedTensorMetadata(slice_sizes, offs[0, :n + 1], offs[1:, :n + 1], sched[:, :width])
