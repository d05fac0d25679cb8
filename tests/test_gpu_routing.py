"""GPU parity: topk, bitmatrix metadata, ragged metadata and routing() vs the CPU oracle (bit-exact integers)."""
import pytest
import torch

from oracle import routing_ref as R
from triton_amd.routing import routing
from triton_amd.tensor import BIT, make_bitmatrix_metadata, make_ragged_tensor_metadata, wrap_torch_tensor
from triton_amd.topk import topk

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_rows", [1, 7, 256, 300])
@pytest.mark.parametrize("n_cols", [13, 32, 128, 200, 811])
@pytest.mark.parametrize("k", [1, 4, 8])
@pytest.mark.parametrize("apply_softmax", [True, False])
def test_topk(n_rows, n_cols, k, apply_softmax, device):
    torch.manual_seed(0)
    x = torch.randn(n_rows, n_cols)
    sp = topk(x.to(device), k, apply_softmax=apply_softmax)
    vals, indx, bits = R.topk_ref(x, k, apply_softmax)
    assert sp.indx.dtype == torch.int16
    assert torch.equal(sp.indx.cpu().int(), indx)
    torch.testing.assert_close(sp.vals.cpu(), vals, rtol=1e-5, atol=1e-6)
    store = sp.mask.storage.data
    assert store.stride() == (1, -(-n_rows // 32) * 32) and tuple(store.shape) == (n_rows, -(-n_cols // 32))
    assert torch.equal(store.cpu().view(torch.int32), bits)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_topk_ties_and_16bit(dtype, device):
    torch.manual_seed(1)
    x = torch.randn(300, 128).to(dtype)  # 16-bit logits collide often: exercises the lower-index-wins rule
    x[:, 64:] = x[:, :64]
    sp = topk(x.to(device), 4)
    vals, indx, bits = R.topk_ref(x, 4)
    assert torch.equal(sp.indx.cpu().int(), indx)
    assert torch.equal(sp.mask.storage.data.cpu().view(torch.int32), bits)
    torch.testing.assert_close(sp.vals.cpu().float(), vals.float(), rtol=2e-2, atol=1e-3)


def test_topk_n_rows_and_provided_indx(device):
    torch.manual_seed(2)
    x = torch.randn(100, 64)
    sp = topk(x.to(device), 4, n_rows=70)
    vals, indx, bits = R.topk_ref(x, 4, n_rows=70)
    assert torch.equal(sp.indx.cpu().int()[:70], indx[:70])
    assert torch.equal(sp.mask.storage.data.cpu().view(torch.int32)[:70], bits[:70])
    y_indx = torch.stack([torch.randperm(64)[:4] for _ in range(100)]).to(torch.int16)
    sp = topk(x.to(device), 4, y_indx=y_indx.to(device))
    vals, indx, bits = R.topk_ref(x, 4, y_indx=y_indx)
    torch.testing.assert_close(sp.vals.cpu(), vals, rtol=1e-5, atol=1e-6)
    assert torch.equal(sp.mask.storage.data.cpu().view(torch.int32), bits)


@pytest.mark.parametrize("n_rows,n_rows_max", [(70, 100), (0, 33), (4097, 5000)])
def test_topk_n_rows_bounds_the_metadata(n_rows, n_rows_max, device):
    """Rows at and beyond `n_rows` are not routed: whatever their index entries hold (here: valid-looking expert
    ids), the histogram and the ordering count the first n_rows rows only and pad with -1
    (tensor_details/bitmatrix.py:138-145 of the reference bounds both stages by bitmatrix.shape[0])."""
    torch.manual_seed(4)
    k, n_cols = 4, 64
    x = torch.randn(n_rows_max, n_cols)
    y_indx = torch.full((n_rows_max, k), 7, dtype=torch.int16, device=device)  # poison: the kernel leaves the tail alone
    vals, indx, bits = R.topk_ref(x, k, n_rows=n_rows)
    y_indx[:n_rows] = indx[:n_rows].to(torch.int16).to(device)
    sp = topk(x.to(device), k, y_indx=y_indx, n_rows=n_rows)
    assert sp.mask.shape[0] == n_rows
    assert torch.equal(sp.indx[n_rows:].cpu(), torch.full((n_rows_max - n_rows, k), 7, dtype=torch.int16))
    ref = R.bitmatrix_metadata_ref(indx[:n_rows], n_cols)
    pad = torch.full(((n_rows_max - n_rows) * k, ), -1, dtype=torch.int32)
    m = sp.mask_metadata
    assert torch.equal(m.col_sum.cpu(), ref.col_sum)
    assert torch.equal(m.col_sorted_indx.cpu(), torch.cat([ref.col_sorted_indx, pad]))
    assert torch.equal(m.row_sorted_indx.cpu(), torch.cat([ref.row_sorted_indx, pad]))
    # without provided indices the tail of indx is whatever the allocation held; the metadata must not depend on it
    sp2 = topk(x.to(device), k, n_rows=n_rows)
    assert torch.equal(sp2.mask_metadata.col_sum.cpu(), ref.col_sum)
    assert torch.equal(sp2.mask_metadata.col_sorted_indx.cpu(), torch.cat([ref.col_sorted_indx, pad]))
    assert torch.equal(sp2.mask_metadata.row_sorted_indx.cpu(), torch.cat([ref.row_sorted_indx, pad]))


@pytest.mark.parametrize("n_rows", [7, 256, 17111])
@pytest.mark.parametrize("n_cols", [13, 32, 128, 811])
@pytest.mark.parametrize("k", [1, 4, 8])
def test_bitmatrix_metadata(n_rows, n_cols, k, device):
    torch.manual_seed(0)
    indx = torch.rand(n_rows, n_cols).argsort(dim=1).int()[:, :k]
    indx = torch.sort(indx, dim=1)[0]
    bm = wrap_torch_tensor(torch.zeros((n_rows, (n_cols + 31) // 32), dtype=torch.int32, device=device).view(torch.uint32),
                           dtype=BIT, shape=(n_rows, n_cols))
    m = make_bitmatrix_metadata(indx.to(device), bm)
    ref = R.bitmatrix_metadata_ref(indx, n_cols)
    assert torch.equal(m.col_sum.cpu(), ref.col_sum)
    assert torch.equal(m.row_sorted_indx.cpu(), ref.row_sorted_indx)
    assert torch.equal(m.col_sorted_indx.cpu(), ref.col_sorted_indx)


def test_bitmatrix_metadata_with_dropped_rows(device):
    torch.manual_seed(3)
    indx = torch.randint(0, 40, (500, 4), dtype=torch.int32)
    indx[350:] = -1
    bm = wrap_torch_tensor(torch.zeros((500, 2), dtype=torch.int32, device=device).view(torch.uint32), dtype=BIT,
                           shape=(500, 40))
    m = make_bitmatrix_metadata(indx.to(device), bm)
    ref = R.bitmatrix_metadata_ref(indx, 40)
    assert torch.equal(m.col_sum.cpu(), ref.col_sum)
    assert torch.equal(m.row_sorted_indx.cpu(), ref.row_sorted_indx)
    assert torch.equal(m.col_sorted_indx.cpu(), ref.col_sorted_indx)


@pytest.mark.parametrize("n_slices", [1, 7, 33, 911, 1025])
def test_ragged_metadata(n_slices, device):
    torch.manual_seed(0)
    max_slice = 200
    total = max_slice * n_slices
    sizes = torch.randint(0, max_slice, (n_slices, ), dtype=torch.int32)
    sizes[torch.randint(0, n_slices, (1, ))] = 0
    m = make_ragged_tensor_metadata(sizes.to(device), total)
    ref = R.ragged_metadata_ref(sizes, total)
    assert torch.equal(m.slice_offs.cpu(), ref.slice_offs)
    assert torch.equal(m.block_offs_data.cpu(), ref.block_offs_data)
    assert torch.equal(m.block_schedule_data.cpu(), ref.block_schedule_data)


@pytest.mark.parametrize("T,E,k", [(4096, 128, 4), (64, 128, 4), (16384, 32, 4), (300, 200, 8), (1, 128, 4), (128, 128, 4),
                                   (129, 128, 4), (100, 13, 1), (33, 512, 8), (64, 200, 8), (16, 64, 64), (255, 40, 2),
                                   (8192, 128, 4), (8193, 128, 4), (4000, 128, 4), (1000, 100, 3), (500, 200, 3),
                                   (2000, 400, 4), (3000, 64, 8)])
def test_routing_configs(T, E, k, device):
    """BASELINE config 2 (T=4096, E=128, k=4) and the routing of configs 4 / 5, plus a run with exact ties.  The small
    row counts run as one launch (top-k and metadata in one workgroup, at most two passes of its 1024 threads over the
    rows: up to 256, 128, 64 or 32 rows for up to 64, 128, 256 or 512 experts); beyond that two launches (top-k with a
    histogram per workgroup, then ordering and tables) while there are at most 128 workgroups of rows that make whole
    chunks of 64 entries (8192 rows of 128 logits; not k = 3 with 200 logits), else four.  The cases sit on both sides
    of each limit."""
    torch.manual_seed(0)
    for ties in (False, True):
        logits = torch.randn(T, E)
        if ties:
            logits[:, E // 2:E // 2 * 2] = logits[:, :E // 2]
        out = routing(logits.to(device), k)
        ref = R.routing_ref(logits, k)
        assert torch.equal(out.indx.cpu().int(), ref["indx"])
        assert torch.equal(out.col_sum.cpu(), ref["col_sum"])
        assert torch.equal(out.scatter_indx.cpu(), ref["scatter_indx"])
        assert torch.equal(out.row_sorted_indx.cpu(), ref["row_sorted_indx"])
        assert torch.equal(out.gather_indx.cpu(), ref["gather_indx"])
        rm = out.ragged_metadata
        assert torch.equal(rm.slice_offs.cpu(), ref["ragged"].slice_offs)
        assert torch.equal(rm.block_offs_data.cpu(), ref["ragged"].block_offs_data)
        assert torch.equal(rm.block_schedule_data.cpu(), ref["ragged"].block_schedule_data)
        torch.testing.assert_close(out.vals.cpu(), ref["vals"], rtol=1e-5, atol=1e-6)
        assert int(out.col_sum.sum()) == T * k


@pytest.mark.parametrize("T,E,k,dt", [(4096, 128, 4, torch.int16), (1500, 96, 4, torch.int32), (30000, 64, 4, torch.int32),
                                      (40000, 64, 4, torch.int16), (700, 1000, 2, torch.int32), (6000, 1000, 2, torch.int32),
                                      (64, 128, 4, torch.int16)])
def test_routing_metadata_entry_point(T, E, k, dt, device):
    """tamd_routing_metadata on given indices with dropped rows (-1) at the end, against the oracle: one launch for the
    smallest case, two launches up to 128 blocks of 1024 entries, three beyond (40000 rows)."""
    from oracle.routing_ref import bitmatrix_metadata_ref, ragged_metadata_ref
    from triton_amd import _lib
    from triton_amd.tensor_details.ragged_tensor import alloc_tables
    torch.manual_seed(5)
    indx = torch.rand(T, E).argsort(dim=1)[:, :k].to(dt)
    indx[T - T // 8:] = -1
    n = T * k
    L = _lib.lib()
    d = indx.to(device)
    col_sum = torch.full((E, ), -7, dtype=torch.int32, device=device)
    combined = torch.full((3 * n, ), -7, dtype=torch.int32, device=device)
    offs, sched, width = alloc_tables(E, n, device)
    ws = torch.empty(L.tamd_bitmatrix_metadata_workspace(n, E), dtype=torch.int32, device=device)
    rc = L.tamd_routing_metadata(_lib.ptr(d), int(dt == torch.int16), n, E, k, _lib.ptr(col_sum), _lib.ptr(combined),
                                 _lib.ptr(combined[n:]), _lib.ptr(combined[2 * n:]), _lib.ptr(offs), offs.stride(0),
                                 _lib.ptr(sched), sched.stride(0), width, _lib.ptr(ws), _lib.stream_ptr(device))
    assert rc == 0
    ref = bitmatrix_metadata_ref(indx, E)
    assert torch.equal(col_sum.cpu(), ref.col_sum)
    assert torch.equal(combined[:n].cpu(), ref.col_sorted_indx)
    assert torch.equal(combined[n:2 * n].cpu(), ref.row_sorted_indx)
    gather = torch.div(ref.col_sorted_indx, k, rounding_mode="trunc")
    assert torch.equal(combined[2 * n:].cpu(), gather)
    rag = ragged_metadata_ref(ref.col_sum, n)
    assert torch.equal(offs[0, :E + 1].cpu(), rag.slice_offs)
    assert torch.equal(offs[1:, :E + 1].cpu(), rag.block_offs_data)
    assert torch.equal(sched[:, :width].cpu(), rag.block_schedule_data)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [100, 1000])
def test_routing_16bit_logits(dtype, T, device):
    """16-bit logits (many exact ties) through the one-launch and the two-launch routing: indices and every table
    bit-exact, gate weights to the output type's rounding."""
    torch.manual_seed(7)
    E, k = 128, 4
    logits = torch.randn(T, E).to(dtype)
    out = routing(logits.to(device), k)
    ref = R.routing_ref(logits, k)
    assert torch.equal(out.indx.cpu().int(), ref["indx"])
    assert torch.equal(out.col_sum.cpu(), ref["col_sum"])
    assert torch.equal(out.scatter_indx.cpu(), ref["scatter_indx"])
    assert torch.equal(out.row_sorted_indx.cpu(), ref["row_sorted_indx"])
    assert torch.equal(out.gather_indx.cpu(), ref["gather_indx"])
    rm = out.ragged_metadata
    assert torch.equal(rm.block_offs_data.cpu(), ref["ragged"].block_offs_data)
    assert torch.equal(rm.block_schedule_data.cpu(), ref["ragged"].block_schedule_data)
    assert out.vals.dtype == dtype
    torch.testing.assert_close(out.vals.cpu().float(), ref["vals"].float(), rtol=2e-2, atol=1e-3)
    sp = out.sparse
    assert torch.equal(sp.mask.storage.data.cpu().view(torch.int32), R.topk_ref(logits, k)[2])
