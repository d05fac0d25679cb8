"""CPU oracle: top-k routing and its index metadata.  Test infrastructure, never shipped.

Restates, with numpy:
  topk_ref                  topk.py:144-185 (topk_torch)
  bitmatrix_metadata_ref    tensor_details/bitmatrix.py:157-168 (torch twin) with
                            the flat-position semantics of the GPU kernel :43-73
  ragged_metadata_ref       tensor_details/ragged_tensor.py:217-253, n_blocks :73-81
  routing_ref               tests/test_distributed.py:201-208
"""
from dataclasses import dataclass

import numpy as np
import torch

BLOCK_SIZES = (16, 32, 64, 128, 256)  # HIP list, ragged_tensor.py:83-85


def topk_ref(x: torch.Tensor, k: int, apply_softmax: bool = True, y_indx=None, n_rows=None):
    """Returns (vals [T,k] x.dtype, indx [T,k] int32, bitmatrix uint32 [T, ceil(E/32)]).

    Selection is by value descending with the lower expert index winning ties
    (stable argsort of -x, topk.py:160); softmax is taken over the k selected
    values in float32 (:171); the result is re-sorted by value (:173-174, a
    no-op for distinct values).  Rows >= n_rows get indx -1 and no bits.
    Bit (t, e) of the matrix is word e//32, bit e%32 (:176-182).  NaN logits
    are unsupported.
    """
    T, E = x.shape
    n_rows = T if n_rows is None else n_rows
    xf = x.to(torch.float32).numpy()
    provided = y_indx is not None
    if provided:
        indx = y_indx.to(torch.int64).numpy().copy()
    else:
        indx = np.argsort(-xf, axis=1, kind="stable")[:, :k]
    vals = np.take_along_axis(xf[:n_rows], indx[:n_rows], axis=1)
    vals = np.concatenate([vals, xf[n_rows:, :k]], axis=0)
    if apply_softmax:
        vals = torch.softmax(torch.from_numpy(vals), dim=-1).to(x.dtype).to(torch.float32).numpy()
    if not provided:
        order = np.argsort(-vals, axis=1, kind="stable")
        vals = np.take_along_axis(vals, order, axis=1)
        indx = np.take_along_axis(indx, order, axis=1)
    indx = indx.astype(np.int32)
    indx[n_rows:] = -1
    words = -(-E // 32)
    bits = np.zeros((T, words), dtype=np.uint32)
    rows = np.repeat(np.arange(n_rows), indx.shape[1])
    cols = indx[:n_rows].reshape(-1).astype(np.int64)
    np.bitwise_or.at(bits, (rows, cols // 32), (np.uint32(1) << (cols % 32).astype(np.uint32)))
    return torch.from_numpy(vals).to(x.dtype), torch.from_numpy(indx), torch.from_numpy(bits.view(np.int32))


@dataclass
class BitmatrixMetadataRef:
    col_sum: torch.Tensor
    col_sorted_indx: torch.Tensor
    row_sorted_indx: torch.Tensor


def bitmatrix_metadata_ref(nonzero_indx: torch.Tensor, n_cols: int) -> BitmatrixMetadataRef:
    """col_sum = histogram of expert ids; col_sorted_indx = flat positions
    (row*k+slot) ordered by expert id, stable; row_sorted_indx[flat] = its rank in
    that order; unused entries are -1.  Entries equal to -1 are skipped.

    The reference's torch twin numbers positions inside the array with the -1
    removed (bitmatrix.py:161-162) while its GPU kernel writes positions of the
    original array (:57, 72-73).  The two coincide whenever the -1 entries form a
    suffix, the only case the reference produces; this oracle uses original
    positions.
    """
    flat = nonzero_indx.reshape(-1).to(torch.int64).numpy()
    n = flat.shape[0]
    valid = np.nonzero(flat != -1)[0]
    order = valid[np.argsort(flat[valid], kind="stable")]
    col_sorted = np.full(n, -1, dtype=np.int32)
    col_sorted[:order.shape[0]] = order
    row_sorted = np.full(n, -1, dtype=np.int32)
    row_sorted[order] = np.arange(order.shape[0], dtype=np.int32)
    col_sum = np.bincount(flat[valid], minlength=n_cols).astype(np.int32)
    assert col_sum.shape[0] == n_cols
    return BitmatrixMetadataRef(torch.from_numpy(col_sum), torch.from_numpy(col_sorted), torch.from_numpy(row_sorted))


def n_blocks(n_slices: int, n_total_rows: int, block_size: int) -> int:
    """Upper bound on the number of row blocks; ragged_tensor.py:73-77."""
    if n_total_rows <= n_slices:
        return n_total_rows
    return n_slices - 1 - ((n_slices - n_total_rows - 1) // block_size)


@dataclass
class RaggedMetadataRef:
    slice_sizes: torch.Tensor
    slice_offs: torch.Tensor
    block_offs_data: torch.Tensor
    block_schedule_data: torch.Tensor


def ragged_metadata_ref(slice_sizes: torch.Tensor, n_total_rows: int) -> RaggedMetadataRef:
    """slice_offs = [0]+cumsum(sizes); per block size b: block_offs =
    [0]+cumsum(ceil(size/b)); block_schedule[b][block_offs[s]+i] = (i<<16)|s for
    i < ceil(size_s/b), padded with -1 to max_n_blocks = n_blocks(.., 16)."""
    sizes = slice_sizes.to(torch.int64).numpy()
    S = sizes.shape[0]
    width = n_blocks(S, n_total_rows, min(BLOCK_SIZES))
    slice_offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    offs_rows, sched_rows = [], []
    for b in BLOCK_SIZES:
        nb = (sizes + b - 1) // b
        offs = np.concatenate([[0], np.cumsum(nb)]).astype(np.int32)
        sched = np.full(width, -1, dtype=np.int32)
        for s in range(S):
            for i in range(int(nb[s])):
                j = int(offs[s]) + i
                if j < width:
                    sched[j] = (i << 16) + s
        offs_rows.append(offs)
        sched_rows.append(sched)
    return RaggedMetadataRef(slice_sizes.to(torch.int32), torch.from_numpy(slice_offs),
                             torch.from_numpy(np.stack(offs_rows)), torch.from_numpy(np.stack(sched_rows)))


def routing_ref(logits: torch.Tensor, k: int):
    """tests/test_distributed.py:201-208.  Returns a dict with every routing output."""
    vals, indx, bits = topk_ref(logits, k, apply_softmax=True)
    meta = bitmatrix_metadata_ref(indx, logits.shape[1])
    ragged = ragged_metadata_ref(meta.col_sum, indx.numel())
    gather = torch.div(meta.col_sorted_indx, k, rounding_mode="trunc")
    return dict(vals=vals, indx=indx, bitmatrix=bits, col_sum=meta.col_sum,
                col_sorted_indx=meta.col_sorted_indx, row_sorted_indx=meta.row_sorted_indx,
                gather_indx=gather, scatter_indx=meta.col_sorted_indx, ragged=ragged)
