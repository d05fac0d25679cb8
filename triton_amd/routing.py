"""`routing(logits, k)`: the composition the reference spells out in
tests/test_distributed.py:201-208 (topk -> histogram / ordering -> ragged
metadata; gather = col_sorted // k, scatter = col_sorted).

One foreign call (`tamd_routing`: one launch at decode sizes, two up to a few thousand rows, else four) writes into
one int32 arena that holds every output and the kernels' workspace; its layout is computed once per shape and the
tensors of the result are views of that arena, built when they are first asked for: at these sizes the host time of
this function is what a step waits for."""
import functools

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
    __slots__ = ("_arena", "_lay", "_bits", "_indx", "_vals", "_cache")

    def __init__(self, arena, lay, bits=None, indx=None, vals=None):
        self._arena, self._lay, self._bits, self._indx, self._vals, self._cache = arena, lay, bits, indx, vals, {}

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
    def indx(self):
        if self._indx is None:
            T, k = self._lay["shape"]
            self._indx = self._view("indx").view(torch.int16)[:T * k].view(T, k)
        return self._indx

    @property
    def vals(self):
        if self._vals is None:
            T, k = self._lay["shape"]
            self._vals = self._view("vals").view(self._lay["vals_dtype"])[:T * k].view(T, k)
        return self._vals

    @property
    def _mask_words(self):
        if self._bits is None:
            T, _ = self._lay["shape"]
            n_words, pad_t = self._lay["bits_shape"]
            self._bits = self._view("bits").view(n_words, pad_t).transpose(0, 1)[:T]
        return self._bits

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
            sp.mask = wrap_torch_tensor(self._mask_words.view(torch.uint32), dtype=BIT, shape=[T, E], shape_max=[T, E])
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


@functools.lru_cache(maxsize=512)
def _arena_layout(T: int, E: int, k: int, vals_dtype: torch.dtype):
    """Where every output of `tamd_routing` (and its workspace) sits in the int32 arena of one call: name -> (offset,
    length) in ints, each part 16-byte aligned.  Depends on the shapes only, so it is built once per shape."""
    n = T * k
    width = RaggedTensorMetadata.max_n_blocks(E, n)
    po = -(-(E + 1) // _PITCH) * _PITCH
    ps = -(-max(width, 1) // _PITCH) * _PITCH
    n_words, pad_t = -(-E // 32), -(-T // 32) * 32
    n_ws = _lib.lib().tamd_bitmatrix_metadata_workspace(n, E)
    per_int = 4 // vals_dtype.itemsize
    lay = {"dims": (E, width, po, ps), "shape": (T, k), "vals_dtype": vals_dtype, "bits_shape": (n_words, pad_t)}
    off = 0
    for name, size in (("col_sum", E), ("col_sorted", n), ("row_sorted", n), ("gather", n), ("offs", 6 * po), ("sched", 5 * ps),
                       ("bits", n_words * pad_t), ("vals", -(-n // per_int)), ("indx", -(-n // 2)), ("ws", n_ws)):
        lay[name] = (off, size)
        off += -(-size // 4) * 4
    lay["total"] = off
    lay["byte_offs"] = {name: 4 * lay[name][0] for name in ("col_sum", "col_sorted", "row_sorted", "gather", "offs", "sched",
                                                            "bits", "vals", "indx", "ws")}
    return lay


def routing(logits: torch.Tensor, n_expts_act: int, y_indx=None) -> RoutingResult:
    if y_indx is not None or logits.stride(1) != 1:
        return _routing_two_calls(logits, n_expts_act, y_indx)
    _lib.require_gpu(logits, "logits")
    assert logits.ndim == 2 and logits.shape[1] < 32768
    T, E = logits.shape
    k = n_expts_act
    dev = logits.device
    code = _lib.dtype_code(logits.dtype)  # (refuses other types before the layout divides by their size)
    lay = _arena_layout(T, E, k, logits.dtype)
    _, width, po, ps = lay["dims"]
    arena = torch.empty(lay["total"], dtype=torch.int32, device=dev)
    base = arena.data_ptr()
    o = lay["byte_offs"]
    rc = _lib.lib().tamd_routing(logits.data_ptr(), code, logits.stride(0), T, E, k, base + o["vals"],
                                 base + o["indx"], base + o["bits"], 1, lay["bits_shape"][1], base + o["col_sum"],
                                 base + o["col_sorted"], base + o["row_sorted"], base + o["gather"], base + o["offs"], po,
                                 base + o["sched"], ps, width, base + o["ws"], _lib.stream_ptr(dev))
    _lib.check(rc, "routing")
    return RoutingResult(arena, lay)


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
