"""GPU parity: induced-subgraph slicing (columns and rows in one pass) vs the oracle,
through the C ABI and through Graph._CAPI_FusionSlicing / _CAPI_BatchFusionSlicing."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import graph_20x5, rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu

ID_DTYPES = [torch.int64, torch.int32]


def _check(got, want):
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy().astype(np.int64), w)


def test_20x5_every_fifth_row(dev):
    # the row slice of the reference's tests/test_rowwise_slicing.cc:7-20 restricted to 3 columns
    indptr, indices = graph_20x5()
    cols = np.array([3, 0, 19], dtype=np.int64)
    rows = np.arange(0, 100, 5, dtype=np.int64)
    got = capi.col_row_slice(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev),
                             to_dev(rows, dev))
    assert np.array_equal(got[0].cpu().numpy(), [0, 1, 2, 3])
    assert np.array_equal(got[1].cpu().numpy(), [3, 0, 19])      # position of rows 15, 0, 95
    assert np.array_equal(got[2].cpu().numpy(), [0, 5, 10])      # first edge of each sliced column
    assert np.array_equal(got[3].cpu().numpy(), [15, 0, 95])
    _check(got, O.col_row_slice(indptr, indices, cols, rows))


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("n_cols,n_rows", [(0, 10), (10, 0), (1, 1), (700, 512), (4096, 4000),
                                           (20000, 3000)])
def test_rmat(dev, n_cols, n_rows, idt):
    n = 1 << 12
    indptr, indices = rmat_csc_np(n, 1 << 17, seed=6)
    rng = np.random.default_rng(n_cols * 7 + n_rows)
    cols = rng.integers(0, n, size=n_cols).astype(np.int64)       # duplicates allowed
    rows = rng.permutation(n)[:n_rows].astype(np.int64)
    got = capi.col_row_slice(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt),
                             to_dev(rows, dev, idt))
    assert got[1].dtype == idt
    want = O.col_row_slice(indptr, indices, cols, rows)
    _check(got, want)
    # the same thing in two steps: column slice, then row slice of the result
    s_ptr, _, s_idx, s_sel = O.slice_columns(indptr, indices, cols, True)
    r_ptr, _, r_idx, r_sel = O.row_slice_csc(s_ptr, s_idx, rows, False)
    assert np.array_equal(want[0], r_ptr) and np.array_equal(want[1], r_idx)
    assert np.array_equal(want[2], r_sel) and np.array_equal(want[3], s_sel[r_sel])


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_hub_columns_span_many_tiles(dev, idt):
    # few columns, each far longer than a workgroup's 2048 positions
    n = 64
    indptr, indices = rmat_csc_np(n, 1 << 18, seed=7)
    cols = np.array([0, 1, 0, 5, 63], dtype=np.int64)
    rows = np.arange(0, n, 3, dtype=np.int64)
    got = capi.col_row_slice(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt),
                             to_dev(rows, dev, idt))
    _check(got, O.col_row_slice(indptr, indices, cols, rows))


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("B", [1, 3, 16])
def test_batched(dev, B, idt):
    n = 1 << 11
    indptr, indices = rmat_csc_np(n, 1 << 16, seed=8)
    rng = np.random.default_rng(B)
    col_sizes = rng.integers(0, 200, size=B)
    row_sizes = rng.integers(0, 600, size=B)
    col_ptr = np.concatenate([[0], np.cumsum(col_sizes)]).astype(np.int64)
    row_ptr = np.concatenate([[0], np.cumsum(row_sizes)]).astype(np.int64)
    cols = rng.integers(0, n, size=col_ptr[-1]).astype(np.int64)
    rows = np.concatenate([rng.permutation(n)[:s] for s in row_sizes] + [np.empty(0, np.int64)]).astype(np.int64)
    got = capi.col_row_slice(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt),
                             to_dev(rows, dev, idt), to_dev(col_ptr, dev), to_dev(row_ptr, dev), n)
    want = O.col_row_slice(indptr, indices, cols, rows, col_ptr, row_ptr, n)
    _check(got, want)
    # batch by batch: rows keep their id, so it is a membership filter of the column slice
    for b in range(B):
        c = cols[col_ptr[b]:col_ptr[b + 1]]
        _, _, s_idx, _ = O.slice_columns(indptr, indices, c, False)
        keep = s_idx[np.isin(s_idx, rows[row_ptr[b]:row_ptr[b + 1]])]
        lo, hi = want[0][col_ptr[b]], want[0][col_ptr[b + 1]]
        assert np.array_equal(want[1][lo:hi], keep)


def test_graph_fusion_slicing_carries_edge_data(dev):
    import graph_sampling_amd as gs
    n = 1 << 10
    indptr, indices = rmat_csc_np(n, 1 << 14, seed=9)
    data = np.random.default_rng(0).random(indices.size).astype(np.float32)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    g._CAPI_SetData(to_dev(data, dev))
    cols = np.random.default_rng(1).permutation(n)[:100].astype(np.int64)
    rows = np.random.default_rng(2).permutation(n)[:300].astype(np.int64)
    sub = g._CAPI_FusionSlicing(to_dev(cols, dev), to_dev(rows, dev))
    want = O.col_row_slice(indptr, indices, cols, rows)
    ptr, idx, _ = sub._CAPI_GetCSC()
    assert np.array_equal(ptr.cpu().numpy(), want[0]) and np.array_equal(idx.cpu().numpy(), want[1])
    assert sub._CAPI_GetNumCols() == 100 and sub._CAPI_GetNumRows() == 300
    assert sub._CAPI_GetNumEdges() == want[1].size
    assert np.array_equal(sub._CAPI_GetData("default").cpu().numpy(), data[want[3]])
    assert np.array_equal(sub._CAPI_GetCols().cpu().numpy(), cols)
    assert np.array_equal(sub._CAPI_GetRows().cpu().numpy(), rows)
    # same subgraph as slicing the columns and then the rows through the plain operators
    two = g._CAPI_Slicing(to_dev(cols, dev), 0, gs._CSC, gs._CSC, False)
    two = two._CAPI_Slicing(to_dev(rows, dev), 1, gs._CSC, gs._CSC, False)
    p2, i2, _ = two._CAPI_GetCSC()
    assert torch.equal(p2, ptr) and torch.equal(i2, idx)
    assert torch.equal(two._CAPI_GetData("default"), sub._CAPI_GetData("default"))


def test_graph_batch_fusion_slicing(dev):
    import graph_sampling_amd as gs
    n = 1 << 10
    indptr, indices = rmat_csc_np(n, 1 << 14, seed=10)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    col_ptr = np.array([0, 50, 50, 120], dtype=np.int64)
    row_ptr = np.array([0, 200, 260, 500], dtype=np.int64)
    rng = np.random.default_rng(3)
    cols = rng.integers(0, n, size=120).astype(np.int64)
    rows = np.concatenate([rng.permutation(n)[:200], rng.permutation(n)[:60], rng.permutation(n)[:240]]).astype(np.int64)
    sub = g._CAPI_BatchFusionSlicing(to_dev(cols, dev), to_dev(col_ptr, dev), to_dev(rows, dev),
                                     to_dev(row_ptr, dev))
    want = O.col_row_slice(indptr, indices, cols, rows, col_ptr, row_ptr, n)
    ptr, idx, _ = sub._CAPI_GetCSC()
    assert np.array_equal(ptr.cpu().numpy(), want[0]) and np.array_equal(idx.cpu().numpy(), want[1])
    assert sub._CAPI_GetNumRows() == n and sub._CAPI_GetNumCols() == 120
