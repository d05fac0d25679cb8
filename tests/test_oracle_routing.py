"""Pins oracle/routing_ref.py: the two worked examples in the reference's docstrings
(tensor_details/bitmatrix.py:11-19, tensor_details/ragged_tensor.py:15-29), torch.topk on tie-free inputs,
crafted ties, and plain python-loop brute force on small inputs."""
import numpy as np
import pytest
import torch

from oracle import routing_ref as RR

# ---------------------------------------------------------------------------- top-k


@pytest.mark.parametrize("T,E,k", [(1, 2, 1), (7, 13, 2), (300, 200, 8), (33, 128, 4), (5, 33, 32)])
def test_topk_matches_torch_topk_without_ties(T, E, k):
    torch.manual_seed(T * 1000 + E)
    x = torch.randn(T, E)
    vals, indx, bits = RR.topk_ref(x, k, apply_softmax=False)
    tv, ti = torch.topk(x, k, dim=1, sorted=True)
    assert torch.equal(vals, tv) and torch.equal(indx, ti.int())
    vs, indx2, _ = RR.topk_ref(x, k, apply_softmax=True)
    assert torch.equal(indx2, indx)
    torch.testing.assert_close(vs, torch.softmax(tv.double(), dim=1).float(), rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(vs.sum(1), torch.ones(T), rtol=1e-5, atol=1e-6)


def test_topk_ties_lower_index_wins():
    # topk_details/_topk_forward.py:27-30 of the reference: equal values are ordered by ascending column.
    x = torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0, 0.0],
                      [5.0, 5.0, 5.0, 5.0, 5.0, 5.0],
                      [0.0, -0.0, 0.0, -1.0, -0.0, 0.0]])
    _, indx, _ = RR.topk_ref(x, 2, apply_softmax=False)
    assert indx.tolist() == [[1, 2], [0, 1], [0, 1]]
    _, indx, _ = RR.topk_ref(x, 4, apply_softmax=False)
    assert indx.tolist() == [[1, 2, 4, 3], [0, 1, 2, 3], [0, 1, 2, 4]]


def test_topk_brute_force_selection():
    rng = np.random.default_rng(3)
    x = torch.from_numpy(rng.integers(-3, 4, size=(40, 17)).astype(np.float32))  # many ties
    k = 5
    _, indx, bits = RR.topk_ref(x, k, apply_softmax=False)
    for t in range(x.shape[0]):
        row = x[t].tolist()
        picked = []
        for _ in range(k):
            best = None
            for e, v in enumerate(row):
                if e in picked:
                    continue
                if best is None or v > row[best]:
                    best = e
            picked.append(best)
        assert indx[t].tolist() == picked
        word = 0
        for e in picked:
            word |= 1 << e
        assert (int(bits[t, 0]) & 0xFFFFFFFF) == word


def test_topk_bitmatrix_words_and_n_rows():
    torch.manual_seed(1)
    x = torch.randn(10, 70)
    _, indx, bits = RR.topk_ref(x, 3, n_rows=6)
    assert bits.shape == (10, 3) and bits.dtype == torch.int32
    assert (indx[6:] == -1).all() and (bits[6:] == 0).all()
    b = bits.numpy().view(np.uint32)
    for t in range(6):
        got = sorted(w * 32 + i for w in range(3) for i in range(32) if (int(b[t, w]) >> i) & 1)
        assert got == sorted(indx[t].tolist())


def test_topk_provided_indices():
    torch.manual_seed(2)
    x = torch.randn(4, 9)
    yi = torch.tensor([[8, 0], [1, 2], [3, 3 + 1], [7, 5]], dtype=torch.int32)
    vals, indx, _ = RR.topk_ref(x, 2, apply_softmax=False, y_indx=yi)
    assert torch.equal(indx, yi)
    assert torch.equal(vals, torch.gather(x, 1, yi.long()))


# ---------------------------------------------------------------------------- bit-matrix metadata


def test_bitmatrix_docstring_example():
    # tensor_details/bitmatrix.py:11-19; nonzeros numbered row-major
    matrix = [[0, 0, 1, 0, 1, 1, 0], [0, 1, 0, 0, 0, 1, 0], [1, 1, 1, 0, 0, 0, 1], [0, 0, 1, 0, 1, 0, 0]]
    flat_cols = [c for row in matrix for c, bit in enumerate(row) if bit]
    m = RR.bitmatrix_metadata_ref(torch.tensor(flat_cols, dtype=torch.int32).view(-1, 1), 7)
    assert m.col_sum.tolist() == [1, 2, 3, 0, 2, 2, 1]
    assert m.col_sorted_indx.tolist() == [5, 3, 6, 0, 7, 9, 1, 10, 2, 4, 8]
    assert m.row_sorted_indx.tolist() == [3, 6, 8, 1, 9, 0, 2, 4, 10, 5, 7]
    # the same matrix as a [4, 4] index array padded with -1: positions are those of the padded array
    padded = torch.full((4, 4), -1, dtype=torch.int32)
    for r, row in enumerate(matrix):
        cols = [c for c, bit in enumerate(row) if bit]
        padded[r, :len(cols)] = torch.tensor(cols, dtype=torch.int32)
    mp = RR.bitmatrix_metadata_ref(padded, 7)
    pos_of_compact = [i for i, v in enumerate(padded.flatten().tolist()) if v != -1]
    assert mp.col_sum.tolist() == [1, 2, 3, 0, 2, 2, 1]
    assert mp.col_sorted_indx.tolist()[:11] == [pos_of_compact[i] for i in m.col_sorted_indx.tolist()]
    assert mp.col_sorted_indx.tolist()[11:] == [-1] * 5
    assert [mp.row_sorted_indx[p].item() for p in pos_of_compact] == m.row_sorted_indx.tolist()


@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (50, 8, 2), (257, 130, 4), (1000, 32, 8)])
def test_bitmatrix_metadata_brute_force_and_invariants(T, E, k):
    rng = np.random.default_rng(T + E)
    indx = np.stack([rng.permutation(E)[:k] if E >= k else rng.integers(0, E, k) for _ in range(T)]).astype(np.int32)
    m = RR.bitmatrix_metadata_ref(torch.from_numpy(indx), E)
    flat = indx.reshape(-1).tolist()
    want_sorted = []
    for e in range(E):
        want_sorted += [i for i, v in enumerate(flat) if v == e]
    assert m.col_sorted_indx.tolist() == want_sorted
    assert m.col_sum.tolist() == [flat.count(e) for e in range(E)]
    assert int(m.col_sum.sum()) == T * k
    assert m.row_sorted_indx[m.col_sorted_indx.long()].tolist() == list(range(T * k))


# ---------------------------------------------------------------------------- ragged metadata


def test_ragged_docstring_example():
    # tensor_details/ragged_tensor.py:15-29.  The docstring's last slice offset ("332") and its 16/64/128
    # schedules contradict its own block_offs; block_offs and the 32-row schedule are self-consistent and pinned.
    r = RR.ragged_metadata_ref(torch.tensor([15, 17, 0, 127], dtype=torch.int32), 159)
    assert r.slice_offs.tolist() == [0, 15, 32, 32, 159]
    offs = {b: r.block_offs_data[i].tolist() for i, b in enumerate(RR.BLOCK_SIZES)}
    assert offs[16] == [0, 1, 3, 3, 11]
    assert offs[32] == [0, 1, 2, 2, 6]
    assert offs[64] == [0, 1, 2, 2, 4]
    assert offs[128] == [0, 1, 2, 2, 3]
    assert offs[256] == [0, 1, 2, 2, 3]
    width = r.block_schedule_data.shape[1]
    assert width == RR.n_blocks(4, 159, 16)
    sched32 = [(v >> 16, v & 0xFFFF) if v != -1 else -1 for v in r.block_schedule_data[1].tolist()]
    assert sched32 == [(0, 0), (0, 1), (0, 3), (1, 3), (2, 3), (3, 3)] + [-1] * (width - 6)


def test_n_blocks_closed_form_is_the_worst_case():
    # ragged_tensor.py:73-77: the bound must be reached by the most fragmenting split of the rows
    # (every slice but one holds a single row) and never exceeded by any split.
    rng = np.random.default_rng(0)
    for S, R, b in [(4, 159, 16), (8, 8, 16), (8, 5, 32), (128, 16384, 16), (3, 100, 64), (1, 77, 16), (5, 6, 16)]:
        bound = RR.n_blocks(S, R, b)
        if R > S:
            worst = [1] * (S - 1) + [R - (S - 1)]
            assert sum(-(-x // b) for x in worst) == bound
        else:
            assert bound == R
        for _ in range(200):
            cuts = np.sort(rng.integers(0, R + 1, size=S - 1))
            sizes = np.diff(np.concatenate([[0], cuts, [R]]))
            assert sum(-(-int(x) // b) for x in sizes) <= bound


@pytest.mark.parametrize("S,R", [(1, 0), (1, 5), (6, 3), (16, 1000), (128, 16384), (33, 700)])
def test_ragged_metadata_brute_force(S, R):
    rng = np.random.default_rng(S * 7 + R)
    cuts = np.sort(rng.integers(0, R + 1, size=S - 1))
    sizes = np.diff(np.concatenate([[0], cuts, [R]])).astype(np.int32)
    r = RR.ragged_metadata_ref(torch.from_numpy(sizes), R)
    acc = 0
    for s in range(S):
        assert r.slice_offs[s].item() == acc
        acc += int(sizes[s])
    assert r.slice_offs[S].item() == R
    width = RR.n_blocks(S, R, 16)
    for bi, b in enumerate(RR.BLOCK_SIZES):
        want = []
        for s in range(S):
            want += [(i << 16) + s for i in range(-(-int(sizes[s]) // b))]
        want = (want + [-1] * width)[:width]
        assert r.block_schedule_data[bi].tolist() == want
        assert r.block_offs_data[bi, -1].item() == sum(-(-int(x) // b) for x in sizes)


# ---------------------------------------------------------------------------- composition


def test_routing_composition():
    torch.manual_seed(0)
    T, E, k = 64, 16, 4
    logits = torch.randn(T, E)
    r = RR.routing_ref(logits, k)
    # tests/test_distributed.py:201-208 of the reference: gather = col_sorted // k, scatter = col_sorted
    assert torch.equal(r["gather_indx"], r["col_sorted_indx"] // k)
    flat_expert = r["indx"].flatten()[r["scatter_indx"].long()]
    assert (flat_expert[1:] >= flat_expert[:-1]).all()  # rows arrive grouped by expert
    # every token appears exactly k times among the gathered rows
    assert torch.bincount(r["gather_indx"].long(), minlength=T).eq(k).all()
    assert r["ragged"].slice_offs[-1].item() == T * k
