"""`routing(logits, k)`: the composition the reference spells out in
tests/test_distributed.py:201-208 (topk -> histogram / ordering -> ragged
metadata; gather = col_sorted // k, scatter = col_sorted), in four launches."""
from dataclasses import dataclass

import torch

from . import _lib
from .tensor import BitmatrixMetadata, RaggedTensorMetadata, SparseMatrix
from .tensor_details.ragged_tensor import alloc_tables
from .topk import topk_forward


@dataclass
class RoutingResult:
    ragged_metadata: RaggedTensorMetadata
    gather_indx: torch.Tensor   # int32 [T*k]: token of the i-th expert-sorted row
    scatter_indx: torch.Tensor  # int32 [T*k]: flat (token*k+slot) of the i-th expert-sorted row
    indx: torch.Tensor          # int16 [T, k]
    vals: torch.Tensor          # [T, k] gate weights (softmax over the k picked)
    col_sum: torch.Tensor       # int32 [E] tokens per expert
    row_sorted_indx: torch.Tensor  # int32 [T*k] inverse of scatter_indx
    sparse: SparseMatrix = None

    def __iter__(self):  # unpack like the reference helper
        yield self.ragged_metadata
        yield self.gather_indx
        yield self.scatter_indx
        yield self.indx

    @property
    def expert_sorted_gate_weights(self):
        """vals in expert-sorted row order: the `gammas` of the down projection."""
        return self.vals.reshape(-1)[self.scatter_indx.long()]


def routing(logits: torch.Tensor, n_expts_act: int, y_indx=None) -> RoutingResult:
    vals, indx, mask = topk_forward(logits, n_expts_act, apply_softmax=True, y_indx=y_indx)
    T, E = logits.shape
    k = n_expts_act
    n = T * k
    dev = logits.device
    L = _lib.lib()
    col_sum = torch.empty(E, dtype=torch.int32, device=dev)
    combined = torch.empty(3 * n, dtype=torch.int32, device=dev)
    offs, sched, width = alloc_tables(E, n, dev)
    ws = torch.empty(L.tamd_bitmatrix_metadata_workspace(n, E), dtype=torch.int32, device=dev)
    rc = L.tamd_routing_metadata(_lib.ptr(indx), 1, n, E, k, _lib.ptr(col_sum), _lib.ptr(combined),
                                 _lib.ptr(combined[n:]), _lib.ptr(combined[2 * n:]), _lib.ptr(offs), offs.stride(0),
                                 _lib.ptr(sched), sched.stride(0), width, _lib.ptr(ws), _lib.stream_ptr(dev))
    _lib.check(rc, "routing")
    meta = RaggedTensorMetadata(col_sum, offs[0, :E + 1], offs[1:, :E + 1], sched[:, :width])
    sparse = SparseMatrix.__new__(SparseMatrix)
    sparse.indx, sparse.vals, sparse.mask = indx, vals, mask
    sparse.mask_metadata = BitmatrixMetadata(col_sum, combined[:n], combined[n:2 * n])
    return RoutingResult(meta, combined[2 * n:], combined[:n], indx, vals, col_sum, combined[n:2 * n], sparse)
