"""Histogram and expert-major ordering of a sparse (token, expert) matrix
(tensor_details/bitmatrix.py of the reference)."""
from dataclasses import dataclass

import torch

from .. import _lib


@dataclass
class BitmatrixMetadata:
    col_sum: torch.Tensor          # int32 [n_cols]: entries per column
    col_sorted_indx: torch.Tensor  # int32 [n]: row-major positions grouped by column, -1 padded
    row_sorted_indx: torch.Tensor  # int32 [n]: inverse of col_sorted_indx


def make_bitmatrix_metadata(nonzero_indx: torch.Tensor, bitmatrix) -> BitmatrixMetadata:
    """`nonzero_indx` [n_rows_max, k] holds the column ids (int16 / int32, -1 = none); `bitmatrix` supplies the
    number of columns and the number of live rows: only rows below `bitmatrix.shape[0]` are counted and placed
    (tensor_details/bitmatrix.py:110-150 of the reference bounds the histogram and the placement the same way),
    the entries of the rows beyond get -1 in both index arrays."""
    assert nonzero_indx.ndim == 2
    _lib.require_gpu(nonzero_indx, "nonzero_indx")
    if nonzero_indx.dtype not in (torch.int16, torch.int32):
        nonzero_indx = nonzero_indx.to(torch.int32)
    indx = nonzero_indx.contiguous()
    n_cols = int(bitmatrix.shape[1])
    n = indx.numel()
    n_live = min(n, max(0, int(bitmatrix.shape[0])) * indx.shape[1])
    dev = indx.device
    L = _lib.lib()
    col_sum = torch.empty(n_cols, dtype=torch.int32, device=dev)
    combined = torch.empty(2 * n, dtype=torch.int32, device=dev)
    if n_live < n:
        combined[n_live:n].fill_(-1)
        combined[n + n_live:].fill_(-1)
    ws = torch.empty(L.tamd_bitmatrix_metadata_workspace(n_live, n_cols), dtype=torch.int32, device=dev)
    rc = L.tamd_bitmatrix_metadata(_lib.ptr(indx), int(indx.dtype == torch.int16), n_live, n_cols, _lib.ptr(col_sum),
                                   _lib.ptr(combined), _lib.ptr(combined[n:]) if n else None, _lib.ptr(ws),
                                   _lib.stream_ptr(dev))
    _lib.check(rc, "make_bitmatrix_metadata")
    return BitmatrixMetadata(col_sum, combined[:n], combined[n:])
