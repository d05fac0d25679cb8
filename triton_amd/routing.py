"""`routing(logits, k)`: the composition the reference spells out in
tests/test_distributed.py:201-208 (topk -> histogram / ordering -> ragged
metadata; gather = col_sorted // k, scatter = col_sorted).

One foreign call (`tamd_routing`: the top-k kernel and the one to three metadata kernels) writes into one int32
arena that holds every integer output and the kernels' workspace; the tensors of the result are views of that
arena, built when they are first asked for: at decode sizes the host time of this function is what a step waits for."""
import torch

from . import _lib
from .tensor import BIT, BitmatrixMetadata, RaggedTensorMetadata, SparseMatrix, wrap_torch_tensor
from .tensor_details.ragged_tensor import _PITCH
from .topk import topk_forward


class RoutingResult:
    """Unpacks like the reference helper into (ragged_metadata, gather_indx, scatter_indx, indx).

    gather_indx  int32 [T*k]: token of the i-th expert-sorted row
    scatter_indx int32 [T*k]: flat (token*k+slot) of the i-th expert-sorted row
    indx int16 [T, k], vals [T, k] gate weights (softmax over the k picked), col_sum int32 [E] tokens per expert,
    row_sorted_indx int32 [T*k] inverse of scatter_indx, sparse: the SparseMatrix a `topk` call returns."""
    __slots__ = ("_arena", "_lay", "_bits", "indx", "vals", "_cache")

    def __init__(self, arena, lay, bits, indx, vals):
        self._arena, self._lay, self._bits, self.indx, self.vals, self._cache = arena, lay, bits, indx, vals, {}

    def _view(self, name):
        v = self._cache.get(name)
        if v is None:
            off, n = self._lay[name]
            v = self._cache[name] = self._arena[off:off + n]
        return v

    col_sum = property(lambda self: self._view("col_sum"))
    scatter_indx = property(lambda self: self._view("col_sorted"))
    row_sorted_indx = property(lambda self: self._view("row_sorted"))
    gather_indx = property(lambda self: self._view("gather"))

    @property
    def ragged_metadata(self):
        md = self._cache.get("ragged")
        if md is None:
            E, width, po, ps = self._lay["dims"]
            offs = self._view("offs").view(6, po)
            sched = self._view("sched").view(5, ps)
            md = self._cache["ragged"] = RaggedTensorMetadata(self.col_sum, offs[0, :E + 1], offs[1:, :E + 1], sched[:, :width])
        return md

    @property
    def sparse(self):
        sp = self._cache.get("sparse")
        if sp is None:
            T, E = self.indx.shape[0], self._lay["dims"][0]
            sp = SparseMatrix.__new__(SparseMatrix)
            sp.indx, sp.vals = self.indx, self.vals
            sp.mask = wrap_torch_tensor(self._bits.view(torch.uint32), dtype=BIT, shape=[T, E], shape_max=[T, E])
            sp.mask_metadata = BitmatrixMetadata(self.col_sum, self.scatter_indx, self.row_sorted_indx)
            self._cache["sparse"] = sp
        return sp

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
    if y_indx is not None or logits.stride(1) != 1:
        return _routing_two_calls(logits, n_expts_act, y_indx)
    _lib.require_gpu(logits, "logits")
    assert logits.ndim == 2 and logits.shape[1] < 32768
    T, E = logits.shape
    k = n_expts_act
    n = T * k
    dev = logits.device
    L = _lib.lib()
    width = RaggedTensorMetadata.max_n_blocks(E, n)
    po = -(-(E + 1) // _PITCH) * _PITCH
    ps = -(-max(width, 1) // _PITCH) * _PITCH
    n_words, pad_t = -(-E // 32), -(-T // 32) * 32
    n_ws = L.tamd_bitmatrix_metadata_workspace(n, E)
    lay, off = {"dims": (E, width, po, ps)}, 0
    for name, size in (("col_sum", E), ("col_sorted", n), ("row_sorted", n), ("gather", n), ("offs", 6 * po), ("sched", 5 * ps),
                       ("bits", n_words * pad_t), ("ws", n_ws)):
        lay[name] = (off, size)
        off += -(-size // 4) * 4  # 16-byte alignment of every part
    arena = torch.empty(off, dtype=torch.int32, device=dev)
    vals = torch.empty((T, k), dtype=logits.dtype, device=dev)
    indx = torch.empty((T, k), dtype=torch.int16, device=dev)
    base = arena.data_ptr()
    p = lambda name: base + 4 * lay[name][0]
    rc = L.tamd_routing(logits.data_ptr(), _lib.dtype_code(logits.dtype), logits.stride(0), T, E, k, vals.data_ptr(),
                        indx.data_ptr(), p("bits"), 1, pad_t, p("col_sum"), p("col_sorted"), p("row_sorted"), p("gather"),
                        p("offs"), po, p("sched"), ps, width, p("ws"), _lib.stream_ptr(dev))
    _lib.check(rc, "routing")
    bo, bn = lay["bits"]
    bits = arena[bo:bo + bn].view(n_words, pad_t).transpose(0, 1)[:T]
    return RoutingResult(arena, lay, bits, indx, vals)


def _routing_two_calls(logits, n_expts_act, y_indx):
    """Provided indices or strided logits: the top-k wrapper, then the metadata entry point."""
    vals, indx, mask = topk_forward(logits, n_expts_act, apply_softmax=True, y_indx=y_indx)
    T, E = logits.shape
    k = n_expts_act
    n = T * k
    dev = logits.device
    L = _lib.lib()
    width = RaggedTensorMetadata.max_n_blocks(E, n)
    po = -(-(E + 1) // _PITCH) * _PITCH
    ps = -(-max(width, 1) // _PITCH) * _PITCH
    n_ws = L.tamd_bitmatrix_metadata_workspace(n, E)
    lay, off = {"dims": (E, width, po, ps)}, 0
    for name, size in (("col_sum", E), ("col_sorted", n), ("row_sorted", n), ("gather", n), ("offs", 6 * po), ("sched", 5 * ps),
                       ("ws", n_ws)):
        lay[name] = (off, size)
        off += -(-size // 4) * 4
    arena = torch.empty(off, dtype=torch.int32, device=dev)
    base = arena.data_ptr()
    p = lambda name: base + 4 * lay[name][0]
    rc = L.tamd_routing_metadata(_lib.ptr(indx), 1, n, E, k, p("col_sum"), p("col_sorted"), p("row_sorted"), p("gather"),
                                 p("offs"), po, p("sched"), ps, width, p("ws"), _lib.stream_ptr(dev))
    _lib.check(rc, "routing")
    return RoutingResult(arena, lay, mask.storage.data.view(torch.int32), indx, vals)
