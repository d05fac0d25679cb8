"""Top-k over experts with optional softmax over the picked k (topk.py of the reference)."""
from typing import Optional, Union

import torch

from . import _lib
from .tensor import BIT, SparseMatrix, Tensor, wrap_torch_tensor


def topk_forward(x, k, apply_softmax=True, dim=1, y_indx=None, n_rows=None):
    """Returns (vals [T,k], indx [T,k] int16, bit matrix Tensor).  The bit matrix
    storage is uint32 [ceil(E/32), pad32(T)] viewed transposed, as in topk.py:52-57."""
    if isinstance(x, Tensor):
        n_rows = x.shape[0] if n_rows is None else n_rows
        x = x.storage.data
    assert x.ndim == 2
    assert dim == 1
    assert x.shape[-1] < 32768
    _lib.require_gpu(x, "x")
    if x.stride(1) != 1:
        x = x.contiguous()
    n_rows_max, n_cols = x.shape
    n_rows = n_rows_max if n_rows is None else int(n_rows)
    dev = x.device
    y_vals = torch.empty((n_rows_max, k), dtype=x.dtype, device=dev)
    provided = y_indx is not None
    if provided:
        assert y_indx.dtype == torch.int16 and y_indx.is_contiguous() and tuple(y_indx.shape) == (n_rows_max, k)
    else:
        y_indx = torch.empty((n_rows_max, k), dtype=torch.int16, device=dev)
    n_words = -(-n_cols // 32)
    bits_store = torch.empty((n_words, -(-n_rows_max // 32) * 32), dtype=torch.int32, device=dev)
    bits = bits_store.transpose(0, 1)[:n_rows_max]
    rc = _lib.lib().tamd_topk_forward(_lib.ptr(x), _lib.dtype_code(x.dtype), x.stride(0), n_rows, n_cols, k,
                                      int(apply_softmax), int(provided), _lib.ptr(y_vals), _lib.ptr(y_indx), k,
                                      _lib.ptr(bits_store), bits.stride(0), bits.stride(1), _lib.stream_ptr(dev))
    _lib.check(rc, "topk")
    bitmatrix = wrap_torch_tensor(bits.view(torch.uint32), dtype=BIT, shape=[n_rows, n_cols],
                                  shape_max=[n_rows_max, n_cols])
    return y_vals, y_indx, bitmatrix


def topk(x: Union[Tensor, torch.Tensor], k: int, apply_softmax: bool = True, dim: int = 1,
         y_indx: Optional[torch.Tensor] = None, n_rows: Optional[int] = None, all_gather: bool = False,
         symm_mem_pool=None) -> SparseMatrix:
    """Sparse matrix equal to `x` with all but the k largest entries of every row
    dropped (values optionally replaced by their softmax).  Ties go to the lower
    column; entries are ordered by value, largest first."""
    if all_gather or symm_mem_pool is not None:
        raise NotImplementedError("all_gather needs more than one GPU")
    vals, indx, mask = topk_forward(x, k, apply_softmax, dim, y_indx, n_rows)
    return SparseMatrix(indx=indx, vals=vals, mask=mask)
