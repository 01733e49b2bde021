"""The reference's gtest suite (tests/*.cc of czkkkkkk/graph_sampling) re-expressed against
torch.classes.gs_classes.Graph / HeteroGraph and torch.ops.gs_ops of this build, plus
end-to-end sampler flows through the Matrix API checked against the CPU oracle."""
import numpy as np
import pytest
import torch

import graph_sampling_amd as gs
from graph_sampling_amd import _COO, _CSC, _CSR, _DCSR
from oracle import oracle as O
from tests.util import rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, scope="module")
def _ops_library():
    gs.load_library()  # torch.ops.gs_ops is used directly below, before any gs.Graph is made


def I(dev):
    return dict(dtype=torch.int64, device=dev)


def F(dev):
    return dict(dtype=torch.float32, device=dev)


def graph20(dev):
    A = gs.Graph(False)
    indptr = torch.arange(0, 21, **I(dev)) * 5
    indices = torch.arange(0, 100, **I(dev))
    A._CAPI_LoadCSC(indptr, indices)
    return A, indptr, indices


def graph12(dev, csr=False):
    A = gs.Graph(False)
    indptr = torch.cat([torch.zeros(10, **I(dev)), torch.arange(0, 3, **I(dev)) * 2])
    indices = torch.arange(1, 4, 2, **I(dev)).repeat(2)
    (A._CAPI_LoadCSR if csr else A._CAPI_LoadCSC)(indptr, indices)
    return A, indptr, indices


# ---------------------------------------------------- test_colwise_slicing.cc
def test_colwise_slicing_test1(dev):
    A, _, _ = graph20(dev)
    sub = A._CAPI_Slicing(torch.arange(0, 3, **I(dev)), 0, _CSC, _CSC, False)
    indptr, indices, _ = sub._CAPI_GetCSC()
    assert indptr.equal(torch.arange(0, 4, **I(dev)) * 5)
    assert indices.equal(torch.arange(0, 15, **I(dev)))


# --------------------------------------------------- test_colwise_sampling.cc
def test_colwise_sampling_test1(dev):
    A, indptr, indices = graph20(dev)
    sub = A._CAPI_Sampling(0, 6, False, _CSC, _CSC)
    p, i, _ = sub._CAPI_GetCSC()
    assert p.equal(indptr) and i.equal(indices)


@pytest.mark.parametrize("fanout", [6, 4])
def test_colwise_sampling_test2_3(dev, fanout):
    A, indptr, indices = graph20(dev)
    sub = A._CAPI_Sampling(0, fanout, True, _CSC, _CSC)
    p, i, _ = sub._CAPI_GetCSC()
    assert p.equal(torch.arange(0, 21, **I(dev)) * fanout)
    assert i.numel() == 20 * fanout and not i[:100].equal(indices[:i.numel()][:100])
    assert torch.unique(i).numel() <= 100


# ------------------------------------------------------------ test_relabel.cc
def test_slicing_relabel_test1(dev):
    A = gs.Graph(False)
    A._CAPI_LoadCSCWithColIds(torch.arange(0, 20, **I(dev)), torch.arange(0, 21, **I(dev)) * 5,
                              torch.arange(0, 100, **I(dev)))
    sub = A._CAPI_Slicing(torch.arange(1, 4, **I(dev)), 0, _CSC, _CSC, True)
    assert (A._CAPI_GetNumCols(), A._CAPI_GetNumRows()) == (20, 100)
    assert (sub._CAPI_GetNumCols(), sub._CAPI_GetNumRows()) == (3, 15)
    p, i, _ = sub._CAPI_GetCSC()
    assert p.equal(torch.arange(0, 4, **I(dev)) * 5) and i.equal(torch.arange(0, 15, **I(dev)))


def _graph12_rows(dev, lo, hi):
    A = gs.Graph(False)
    indptr = torch.cat([torch.zeros(10, **I(dev)), torch.arange(0, 3, **I(dev)) * 2])
    A._CAPI_LoadCSC(indptr, torch.arange(lo, hi, **I(dev)).repeat(2))
    return A


def test_slicing_relabel_test2_dcsr(dev):
    # tests/test_relabel.cc:28-52
    A = _graph12_rows(dev, 5, 7)
    A._CAPI_CSC2DCSR()
    sub = A._CAPI_Slicing(torch.arange(5, 6, **I(dev)), 1, _DCSR, _CSR, True)
    assert (A._CAPI_GetNumCols(), A._CAPI_GetNumRows()) == (12, 12)
    assert (sub._CAPI_GetNumCols(), sub._CAPI_GetNumRows()) == (2, 1)
    p, i, _ = sub._CAPI_GetCSR()
    assert p.numel() == 2 and i.equal(torch.arange(0, 2, **I(dev)))
    assert sub._CAPI_GetCols().equal(torch.arange(10, 12, **I(dev)))


def test_rowwise_slicing_test2_dcsr(dev):
    # tests/test_rowwise_slicing.cc:22-38
    A = _graph12_rows(dev, 5, 7)
    A._CAPI_CSC2DCSR()
    sub = A._CAPI_Slicing(torch.arange(5, 6, **I(dev)), 1, _DCSR, _CSR, False)
    p, i, _ = sub._CAPI_GetCSR()
    assert p.numel() == 2 and i.equal(torch.arange(10, 12, **I(dev)))
    # a row that is not stored comes back as an empty row
    sub = A._CAPI_Slicing(torch.tensor([0, 6, 11], **I(dev)), 1, _DCSR, _CSR, False)
    p, i, _ = sub._CAPI_GetCSR()
    assert p.tolist() == [0, 0, 2, 2] and i.equal(torch.arange(10, 12, **I(dev)))


def test_csc2dcsr_test1(dev):
    # tests/test_format_transform.cc:100-116
    A = gs.Graph(False)
    indptr = torch.cat([torch.zeros(10, **I(dev)), torch.arange(0, 3, **I(dev)) * 2])
    A._CAPI_LoadCSC(indptr, torch.arange(1, 4, 2, **I(dev)).repeat(2))
    A._CAPI_CSC2DCSR()
    p, i, _ = A._CAPI_GetCSR()
    assert p.numel() == 3 and p.tolist() == [0, 2, 4]
    assert i.equal(torch.arange(10, 12, **I(dev)).repeat(2))
    assert A._CAPI_GetValidRows().equal(torch.arange(1, 4, 2, **I(dev)))
    with pytest.raises(RuntimeError, match="Require CSR, get DCSR instead"):
        A._CAPI_CreateSparseFormat(_CSR)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_doubly_compressed_round_trip_and_edge_ops(dev, idt):
    """DCSC built from a COO with many empty columns: conversion back, column slice, sums,
    divide and SDDMM agree with the same graph held as a plain CSC."""
    from oracle import oracle as O
    from tests.util import to_dev
    rng = np.random.default_rng(0)
    n, E = 5000, 3000
    row = rng.integers(0, n, size=E).astype(np.int64)
    col = rng.integers(0, 40, size=E).astype(np.int64) * 100      # 40 columns own all edges
    w = rng.random(E).astype(np.float32)

    def make():
        g = gs.Graph(False)
        g._CAPI_LoadCOO(to_dev(row, dev, idt), to_dev(col, dev, idt))
        g._CAPI_SetMetadata(None, None, n, n)
        g._CAPI_SetData(to_dev(w, dev))
        return g

    d, c = make(), make()
    d._CAPI_CreateSparseFormat(8)      # _DCSC
    c._CAPI_CreateSparseFormat(_CSC)
    dp, di, _ = d._CAPI_GetCSC()
    w_ptr, w_val, w_perm = O.coo2csc(col, row, n, False)
    stored = np.flatnonzero(np.diff(w_ptr))
    assert np.array_equal(dp.cpu().numpy(), np.concatenate([w_ptr[stored], [E]]))
    assert np.array_equal(di.cpu().numpy(), w_val)
    assert np.array_equal(d._CAPI_GetValidCols().cpu().numpy(), stored)
    # sums over columns land at the stored columns' ids
    assert torch.equal(d._CAPI_Sum(0, 2, 8), c._CAPI_Sum(0, 2, _CSC))
    div = torch.rand(n, device=dev) + 0.5
    assert torch.equal(d._CAPI_Divide(div, 0, 8)._CAPI_GetData("col"),
                       c._CAPI_Divide(div, 0, _CSC)._CAPI_GetData("col"))
    # column slice: stored, not stored and repeated columns
    ids = to_dev(np.array([100, 101, 3900, 100, 4999, 0]), dev, idt)
    sd = d._CAPI_Slicing(ids, 0, 8, _CSC + _COO, False)
    sc = c._CAPI_Slicing(ids, 0, _CSC, _CSC + _COO, False)
    for a, b in zip(sd._CAPI_GetCSC()[:2], sc._CAPI_GetCSC()[:2]):
        assert torch.equal(a, b)
    assert torch.equal(sd._CAPI_GetData("default"), sc._CAPI_GetData("default"))
    # SDDMM u_add_v on the compressed format uses the stored columns' ids for the v side
    lhs, rhs = torch.rand(n, 1, device=dev), torch.rand(n, 1, device=dev)
    out_d, out_c = torch.zeros(E, 1, device=dev), torch.zeros(E, 1, device=dev)
    d._CAPI_SDDMM("add", lhs, rhs, out_d, 0, 2, 8)
    c._CAPI_SDDMM("add", lhs, rhs, out_c, 0, 2, _CSC)
    assert torch.equal(out_d, out_c)
    # back to COO: the stored columns' ids, not their positions
    e = gs.Graph(False)
    e._CAPI_LoadCOO(to_dev(row, dev, idt), to_dev(col, dev, idt))
    e._CAPI_SetMetadata(None, None, n, n)
    e._CAPI_CreateSparseFormat(8)
    p, i, _ = e._CAPI_GetCSC()
    f = gs.Graph(False)
    f._CAPI_LoadCSC(p, i)
    f._CAPI_SetMetadata(None, None, n, n)
    f._CAPI_SetValidCols(e._CAPI_GetValidCols())
    r2, c2 = f._CAPI_GetBatchCOO()
    assert np.array_equal(c2.cpu().numpy(), np.sort(col, kind="stable"))
    assert np.array_equal(r2.cpu().numpy(), w_val)


# ---------------------------------------------------- test_rowwise_slicing.cc
def test_rowwise_slicing_test1(dev):
    A, _, _ = graph20(dev)
    sub = A._CAPI_Slicing(torch.arange(0, 100, 5, **I(dev)), 1, _CSC, _CSC, False)
    p, i, _ = sub._CAPI_GetCSC()
    assert p.equal(torch.arange(21, **I(dev))) and i.equal(torch.arange(20, **I(dev)))


# ------------------------------------------------------- test_listsampling.cc
def test_list_sampling(dev):
    data = torch.arange(1000, **I(dev))
    sel, idx = torch.ops.gs_ops._CAPI_ListSampling(data, 2000, False)
    assert sel.equal(data)
    sel, idx = torch.ops.gs_ops._CAPI_ListSampling(data, 2000, True)
    assert sel.numel() == 2000 and not sel[:1000].equal(data) and torch.unique(sel).numel() <= 1000
    sel, idx = torch.ops.gs_ops._CAPI_ListSampling(data, 999, False)
    assert sel.numel() == 999 and torch.unique(sel).numel() == 999


# ------------------------------------------------------ test_graph_compute.cc
def test_graph_sum_test1_to_4(dev):
    A, _, _ = graph20(dev)
    assert A._CAPI_Sum(0, 1, _CSC).equal(torch.ones(20, **F(dev)) * 5)
    assert A._CAPI_Sum(0, 2, _CSC).equal(torch.ones(20, **F(dev)) * 5)
    data = torch.arange(1, 6, **F(dev))
    A._CAPI_SetData(data.repeat(20))
    assert A._CAPI_Sum(0, 1, _CSC).equal(data.sum().repeat(20))
    assert A._CAPI_Sum(0, 2, _CSC).equal(data.pow(2).sum().repeat(20))


@pytest.mark.parametrize("fmt", [_CSR, _COO])
def test_graph_sum_test5_6(dev, fmt):
    A, _, _ = graph12(dev)
    A._CAPI_SetData(torch.arange(3, 7, **F(dev)))
    if fmt == _CSR:
        A._CAPI_CSC2CSR()
    expected = torch.tensor([0, 8, 0, 10] + [0] * 8, **F(dev))
    assert A._CAPI_Sum(1, 1, fmt).equal(expected)


def test_graph_sum_test7(dev):
    A, _, _ = graph12(dev)
    A._CAPI_SetData(torch.arange(3, 7, **F(dev)))
    A._CAPI_Slicing(torch.arange(10, 12, **I(dev)), 0, _CSC, _CSC, False)
    assert A._CAPI_Sum(1, 1, _CSR).equal(torch.tensor([0, 8, 0, 10] + [0] * 8, **F(dev)))


@pytest.mark.parametrize("fmt", [_CSC, _COO])
def test_graph_div(dev, fmt):
    A, _, _ = graph20(dev)
    if fmt == _CSC:
        out = A._CAPI_Divide(torch.ones(20, **F(dev)) * 10, 0, _CSC)._CAPI_GetData("default")
        assert torch.isclose(out, torch.ones(100, **F(dev)) / 10).all()
    divisor = torch.arange(1, 21, **F(dev))
    out = A._CAPI_Divide(divisor, 0, fmt)._CAPI_GetData("default")
    assert torch.isclose(out, torch.repeat_interleave(1 / divisor, 5)).all()


@pytest.mark.parametrize("fmt", [_CSC, _COO])
def test_graph_normalize_test1_to_3(dev, fmt):
    A, _, _ = graph20(dev)
    out = A._CAPI_Divide(A._CAPI_Sum(0, 1, _CSC), 0, _CSC)._CAPI_GetData("default")
    assert torch.isclose(out, torch.ones(100, **F(dev)) / 5).all()
    data = torch.arange(1, 6, **F(dev))
    A._CAPI_SetData(data.repeat(20))
    out = A._CAPI_Divide(A._CAPI_Sum(0, 1, fmt), 0, fmt)._CAPI_GetData("default")
    assert torch.isclose(out, (data / data.sum()).repeat(20)).all()


def test_graph_normalize_test4(dev):
    A, _, _ = graph12(dev)
    data = torch.arange(3, 7, **F(dev))
    A._CAPI_SetData(data)
    g = A._CAPI_Slicing(torch.arange(10, 12, **I(dev)), 0, _CSC, _CSC, False)
    g = g._CAPI_Divide(g._CAPI_Sum(1, 1, _CSR), 1, _CSR)
    expected = torch.flatten(data.reshape(2, 2) / data.reshape(2, 2).sum(0))
    assert g._CAPI_GetData("default").equal(expected)


@pytest.mark.parametrize("fmt", [_CSC, _COO])
def test_graph_normalize_test5_6(dev, fmt):
    A, _, _ = graph12(dev, csr=True)
    data = torch.arange(3, 7, **F(dev))
    A._CAPI_SetData(data)
    g = A._CAPI_Slicing(torch.arange(10, 12, **I(dev)), 1, _CSR, _CSR, False)
    g = g._CAPI_Divide(torch.ones(2, **F(dev)), 1, _CSR)
    g = g._CAPI_Divide(g._CAPI_Sum(0, 1, fmt), 0, fmt)
    expected = torch.flatten(data.reshape(2, 2) / data.reshape(2, 2).sum(0))
    assert g._CAPI_GetData("default").equal(expected)


def test_normalize_method(dev):
    A, _, _ = graph20(dev)
    data = torch.arange(1, 6, **F(dev))
    A._CAPI_SetData(data.repeat(20))
    out = A._CAPI_Normalize(0, _CSC)._CAPI_GetData("default")
    assert torch.isclose(out, (data / data.sum()).repeat(20)).all()


# ---------------------------------------------------------------- test_sddmm.cc
@pytest.mark.parametrize("fmt", [_COO, _CSR, _CSC])
def test_sddmm_add_coo_loaded(dev, fmt):
    A = gs.Graph(False)
    r = torch.arange(0, 100, **I(dev))
    A._CAPI_LoadCOO(r, r.clone())
    f = torch.arange(0, 100, **F(dev))
    out = torch.zeros(100, **F(dev))
    A._CAPI_SDDMM("add", f, f.clone(), out, 0, 2, fmt)
    assert out.equal(f * 2)


@pytest.mark.parametrize("fmt", [_COO, _CSR, _CSC])
@pytest.mark.parametrize("with_col_ids", [False, True])
def test_sddmm_add_csc_loaded(dev, fmt, with_col_ids):
    if fmt == _CSR and not with_col_ids:
        pytest.skip("LoadCSC sets num_rows = num_cols = 20 while rows reach 99: no valid CSR")
    A = gs.Graph(False)
    indptr = torch.arange(0, 21, **I(dev)) * 5
    indices = torch.arange(0, 100, **I(dev))
    if with_col_ids:
        A._CAPI_LoadCSCWithColIds(torch.arange(2, 22, **I(dev)), indptr, indices)
    else:
        A._CAPI_LoadCSC(indptr, indices)
    lhs = torch.arange(0, 100, **F(dev))
    rhs = torch.arange(0, 20, **F(dev))
    out = torch.zeros(100, **F(dev))
    A._CAPI_SDDMM("add", lhs, rhs, out, 0, 2, fmt)
    assert out.equal(lhs + torch.repeat_interleave(rhs, 5))


def test_sddmm_unknown_op_raises(dev):
    A, _, _ = graph20(dev)
    with pytest.raises(RuntimeError, match="Unsupported SpMM/SDDMM binary operator"):
        A._CAPI_SDDMM("pow", torch.zeros(100, **F(dev)), torch.zeros(20, **F(dev)),
                      torch.zeros(100, **F(dev)), 0, 2, _COO)


# ------------------------------------------------------ test_format_transform.cc
def test_csc2csr_test1_and_csr2csc(dev):
    A = gs.Graph(True)
    col_ids = torch.arange(0, 20, **I(dev))
    indptr = torch.arange(0, 21, **I(dev)) * 5
    indices = torch.arange(0, 100, **I(dev))
    col = torch.repeat_interleave(col_ids, 5)
    A._CAPI_LoadCSCWithColIds(col_ids, indptr, indices)
    A._CAPI_CSC2CSR()
    _, _, _, row, c = A._CAPI_COOMetadata()
    assert row.equal(indices) and c.equal(col)
    assert A._CAPI_GetNumRows() == 100
    assert A._CAPI_GetCOORows(True).equal(indices)
    assert A._CAPI_AllValidNode().equal(indices)
    A._CAPI_CSR2CSC()
    p, i, _ = A._CAPI_GetCSC()
    assert p.equal(indptr) and i.equal(indices)


def test_csc2csr_test2(dev):
    A = gs.Graph(True)
    col_ids = torch.arange(0, 21, **I(dev))
    indptr = torch.cat([torch.zeros(1, **I(dev)), torch.arange(0, 21, **I(dev))]) * 5
    indices = torch.arange(2, 102, **I(dev))
    A._CAPI_LoadCSCWithColIds(col_ids, indptr, indices)
    A._CAPI_CSC2CSR()
    assert A._CAPI_GetNumRows() == 102
    assert A._CAPI_AllValidNode().equal(torch.arange(0, 102, **I(dev)))
    _, _, _, row, c = A._CAPI_COOMetadata()
    assert c.equal(torch.repeat_interleave(torch.arange(1, 21, **I(dev)), 5))


def test_csc2csr_test3_eids(dev):
    A, _, _ = graph12(dev)
    A._CAPI_SetData(torch.arange(3, 7, **F(dev)))
    A._CAPI_CSC2CSR()
    # the CSR is reachable through Sum / GetData('row'); its edge order is the stable sort by row
    assert A._CAPI_GetData("row").equal(torch.tensor([3, 5, 4, 6], **F(dev)))
    assert A._CAPI_GetValidRows().equal(torch.tensor([1, 3], **I(dev)))


# -------------------------------------------------- test_hetero_random_walk.cc
def _hetero(dev, indptr2, indices2):
    g1, g2 = gs.Graph(False), gs.Graph(False)
    g1._CAPI_LoadCSC(torch.tensor([0, 0, 1, 2, 3], **I(dev)), torch.tensor([0, 1, 2], **I(dev)))
    g2._CAPI_LoadCSC(torch.tensor(indptr2, **I(dev)), torch.tensor(indices2, **I(dev)))
    hg = gs.HeteroGraph()
    hg._CAPI_LoadFromHomo(["user", "item"], [("user", "follow", "user"), ("user", "view", "item")], [g1, g2])
    return hg


def test_random_walk_one_path(dev):
    hg = _hetero(dev, [0, 1, 2, 3], [0, 1, 2])
    seeds = torch.tensor([2, 1], **I(dev))
    paths = hg._CAPI_MetapathRandomWalkFused(seeds, ["view", "follow", "follow"])
    assert paths.shape == (2, 4)
    assert paths.reshape(-1, 2).cpu().equal(torch.tensor([[2, 1], [2, 1], [1, 0], [0, -1]]))


def test_random_walk_multi_path(dev):
    hg = _hetero(dev, [0, 1, 3, 5], [0, 0, 1, 2, 3])
    seeds = torch.tensor([2, 2, 1, 1, 0], **I(dev))
    metapath = ["view", "follow", "follow"]
    tr = hg._CAPI_MetapathRandomWalkFused(seeds, metapath).reshape(-1, 5).cpu().numpy()
    for w in range(5):
        for t, et in enumerate(metapath):
            g = hg._CAPI_GetHomoGraph(et)
            p, i = [x.cpu().numpy() for x in g._CAPI_GetCSC()[:2]]
            s, d = tr[t, w], tr[t + 1, w]
            assert d == -1 or d in i[p[s]:p[s + 1]]


# ------------------------------------------------------ end-to-end sampler flows
def _rmat_matrix(dev, n_log, e_log, seed, with_data=False):
    indptr, indices = rmat_csc_np(1 << n_log, 1 << e_log, seed=seed)
    m = gs.Matrix()
    data = None
    if with_data:
        data = (1.0 - np.random.default_rng(seed).random(indices.size)).astype(np.float32)
    m.load_csc(to_dev(indptr, dev), to_dev(indices, dev), None if data is None else to_dev(data, dev))
    return m, indptr, indices, data


@pytest.mark.parametrize("algo", [0, 1])
def test_graphsage_fused_flow_matches_oracle(dev, algo):
    """examples/graphsage: fused_columnwise_slicing_sampling + relabel per layer."""
    m, indptr, indices, _ = _rmat_matrix(dev, 13, 17, 1)
    torch.ops.gs_ops._CAPI_SetSampleAlgo(algo)
    try:
        seeds = np.random.default_rng(0).permutation(1 << 13)[:256].astype(np.int64)
        d_seeds = to_dev(seeds, dev)
        for layer, fanout in enumerate([10, 5]):
            gs.set_seed(1000 + layer)
            sub = m.fused_columnwise_slicing_sampling(d_seeds, fanout, False)
            block = sub.to_dgl_block()
            sp, _, rows, sel = O.sample_uniform(indptr, indices, seeds, fanout, False, seed=1000 + layer,
                                                with_coo=False, algo=algo)
            frontier, (rel,) = O.relabel([seeds, rows], [rows])
            assert block.format == "csc" and block.num_dst_nodes() == seeds.size
            assert np.array_equal(block.csc()[0].cpu().numpy(), sp)
            assert np.array_equal(block.csc()[1].cpu().numpy(), rel)
            assert np.array_equal(block.srcdata["_ID"].cpu().numpy(), frontier)
            assert np.array_equal(block.dstdata["_ID"].cpu().numpy(), seeds)
            assert block.num_src_nodes() == frontier.size and block.num_edges() == rel.size
            assert np.array_equal(block.in_degrees().cpu().numpy(), np.diff(sp))
            src, dst = block.edges()  # COO view made by the library's CSC -> COO kernel
            assert np.array_equal(src.cpu().numpy(), rel)
            assert np.array_equal(dst.cpu().numpy(), np.repeat(np.arange(seeds.size), np.diff(sp)))
            assert np.array_equal(sub.all_indices().cpu().numpy(), frontier)
            assert np.array_equal(sub.row_indices().cpu().numpy(), rows)
            seeds, d_seeds = frontier, block.srcdata["_ID"]
    finally:
        torch.ops.gs_ops._CAPI_SetSampleAlgo(0)


def test_graphsage_nonfused_flow_matches_oracle(dev):
    """A[:, seeds] -> columnwise_sampling -> all_indices / to_dgl_block (COO path)."""
    m, indptr, indices, data = _rmat_matrix(dev, 12, 16, 2, with_data=True)
    seeds = np.random.default_rng(1).permutation(1 << 12)[:200].astype(np.int64)
    sliced = m[:, to_dev(seeds, dev)]
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    assert np.array_equal(sliced.row_indices().cpu().numpy(), si)
    assert np.array_equal(sliced.get_data().cpu().numpy(), data[sel])
    gs.set_seed(77)
    sampled = sliced.columnwise_sampling(7, False)
    # sampling runs over every column of the sliced CSC (built from the column-sorted COO)
    sp2, coo2, si2, sel2 = O.sample_uniform(sp, si, None, 7, False, seed=77)
    block = sampled.to_dgl_block()
    frontier, (rel_col, rel_row) = O.relabel([seeds, si2], [seeds[coo2], si2])
    assert block.format == "coo"
    assert np.array_equal(block.edges()[0].cpu().numpy(), rel_row)
    assert np.array_equal(block.edges()[1].cpu().numpy(), rel_col)
    assert np.array_equal(block.srcdata["_ID"].cpu().numpy(), frontier)
    assert np.array_equal(sampled.get_data().cpu().numpy(), data[sel][sel2])
    assert np.array_equal(block.edata["w"].cpu().numpy(), data[sel][sel2])
    # by-destination view and the sparse matrix a model multiplies with: A[dst, src] = sum of w
    ptr, src, order = block.csc()
    assert ptr.numel() == seeds.size + 1 and int(ptr[-1]) == rel_row.size
    dense = np.zeros((seeds.size, frontier.size))
    np.add.at(dense, (rel_col, rel_row), data[sel][sel2].astype(np.float64))
    feat = torch.randn(frontier.size, 8, device=dev)
    np.testing.assert_allclose((block.adj() @ feat).cpu().numpy(),
                               dense @ feat.cpu().numpy().astype(np.float64), rtol=1e-4, atol=1e-5)


def test_weighted_sampling_flow(dev):
    m, indptr, indices, data = _rmat_matrix(dev, 11, 15, 3, with_data=True)
    gs.set_seed(5)
    sub = m.columnwise_sampling(6, False, bias=to_dev(data, dev))
    want = O.sample_weighted(indptr, indices, data, None, 6, seed=5)
    _, _, _, row, col = sub._graph._CAPI_COOMetadata()
    assert np.array_equal(row.cpu().numpy(), want[2]) and np.array_equal(col.cpu().numpy(), want[1])


def test_ladies_flow_matches_oracle(dev):
    """examples/ladies: U = P[:, seeds]; prob = U.sum(1, powk=2); weighted list sampling of rows;
    subU = U[nodes, :]; divide by prob; normalise columns; relabel."""
    m, indptr, indices, data = _rmat_matrix(dev, 12, 16, 4, with_data=True)
    N = 1 << 12
    seeds = np.random.default_rng(2).permutation(N)[:128].astype(np.int64)
    U = m[:, to_dev(seeds, dev)]
    prob = U.sum(axis=1, powk=2)
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    want_prob = O.coo_sum(si, None, data[sel], 2, N)
    np.testing.assert_allclose(prob.cpu().numpy(), want_prob, rtol=1e-5)

    row_ids = U.row_ids(remove_isolated=False)
    assert np.array_equal(row_ids.cpu().numpy(), np.arange(N))
    gs.set_seed(31)
    selected, idx = torch.ops.gs_ops._CAPI_ListSamplingWithProbs(row_ids, prob, 64, False)
    w_sel, w_idx = O.list_sample_weighted(np.arange(N), prob.cpu().numpy(), 64, seed=31)
    assert np.array_equal(idx.cpu().numpy(), w_idx) and np.array_equal(selected.cpu().numpy(), w_sel)
    assert (want_prob[w_idx] > 0).all()

    nodes = torch.cat([to_dev(seeds, dev), selected]).unique()
    subU = U[nodes, :]
    h_nodes = nodes.cpu().numpy()
    # row slice on the CSR of U: edges of U whose row is in nodes, in CSR (row-major) order
    r_ip, r_col, r_perm = O.coo2csc(si, coo, N, False)
    s_ip, s_row, s_col, s_sel = O.slice_columns(r_ip, r_col, h_nodes)
    assert subU.get_num_rows() == h_nodes.size and subU.get_num_edges() == s_col.size
    w_data = data[sel][r_perm][s_sel]
    assert np.array_equal(subU.get_data().cpu().numpy(), w_data)

    div = subU.divide(prob[nodes], axis=1)
    w_div = w_data / want_prob[h_nodes][s_row]
    np.testing.assert_allclose(div.get_data().cpu().numpy(), w_div, rtol=1e-5)
    norm = div.normalize(axis=0)
    col_sum = np.bincount(s_col, weights=w_div.astype(np.float64), minlength=seeds.size)
    np.testing.assert_allclose(norm.get_data().cpu().numpy(), w_div / col_sum[s_col], rtol=1e-4)

    block = subU.to_dgl_block()
    frontier, (rel_col, rel_row) = O.relabel([seeds, h_nodes[s_row]], [seeds[s_col], h_nodes[s_row]])
    assert np.array_equal(block.srcdata["_ID"].cpu().numpy(), frontier)
    assert np.array_equal(block.edges()[0].cpu().numpy(), rel_row)
    assert np.array_equal(block.edges()[1].cpu().numpy(), rel_col)


@pytest.mark.parametrize("ids", ["increasing", "shuffled", "repeated"])
def test_row_slice_of_a_column_slice_is_the_same_by_filter_and_by_sorted_rows(dev, ids):
    """`U[nodes, :]` of a column slice (a COO) filters the COO and sorts the kept edges when the
    ids increase, and goes through the CSR of all of U otherwise (or when ordered sums have
    built that CSR): the same edges in the same order with the same data, and both equal the
    oracle's row slice of U's CSR (src/graph.cc:258-283)."""
    m, indptr, indices, data = _rmat_matrix(dev, 12, 16, 9, with_data=True)
    N = 1 << 12
    rng = np.random.default_rng(3)
    seeds = rng.permutation(N)[:200].astype(np.int64)
    nodes = np.sort(rng.permutation(N)[:700]).astype(np.int64)
    if ids == "shuffled":
        nodes = rng.permutation(nodes)
    elif ids == "repeated":
        nodes = np.sort(np.concatenate([nodes, nodes[:50]]))
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    r_ip, r_col, r_perm = O.coo2csc(si, coo, N, False)
    s_ip, s_row, s_col, s_sel = O.slice_columns(r_ip, r_col, nodes)
    got = []
    for ordered in (False, True):
        gs.set_ordered_sums(ordered)
        try:
            U = m[:, to_dev(seeds, dev)]
            U.sum(axis=1)  # ordered: builds the CSR of U, which the slice then uses
            sub = U[to_dev(nodes, dev), :]
        finally:
            gs.set_ordered_sums(False)
        assert sub.get_num_rows() == nodes.size and sub.get_num_edges() == s_col.size
        assert np.array_equal(sub.get_data().cpu().numpy(), data[sel][r_perm][s_sel])
        block = sub.to_dgl_block()
        got.append([t.cpu().numpy() for t in (block.srcdata["_ID"], *block.edges(), block.edata["w"])])
    for a, b in zip(*got):
        assert np.array_equal(a, b)


def test_sum_over_the_rows_of_a_column_slice_adds_edge_by_edge_or_in_order(dev):
    """`U.sum(axis=1)` of a column slice held as a COO adds straight off the COO (float atomics)
    unless ordered sums are on (CSR of U, one row after the other): the oracle's sums to 1e-5
    either way, and with ordered sums the same bits on every run."""
    m, indptr, indices, data = _rmat_matrix(dev, 14, 19, 6, with_data=True)
    N = 1 << 14
    seeds = np.random.default_rng(8).permutation(N)[:6000].astype(np.int64)
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    assert si.size >= 1 << 17  # enough edges for the sum through bins
    want = O.coo_sum(si, None, data[sel], 2, N)
    runs = []
    for ordered in (False, True, True):
        gs.set_ordered_sums(ordered)
        try:
            prob = m[:, to_dev(seeds, dev)].sum(axis=1, powk=2)
        finally:
            gs.set_ordered_sums(False)
        np.testing.assert_allclose(prob.cpu().numpy(), want, rtol=1e-5)
        runs.append(prob)
    assert torch.equal(runs[1], runs[2])


def test_fastgcn_coo_row_slicing_flow(dev):
    """examples/fastgcn/unbatching_training.py:18-31: _CAPI_slicing(selected, 1, _COO, _COO, False)."""
    m, indptr, indices, _ = _rmat_matrix(dev, 11, 15, 5)
    seeds = np.random.default_rng(3).permutation(1 << 11)[:100].astype(np.int64)
    U = m[:, to_dev(seeds, dev)]
    selected = np.random.default_rng(4).permutation(1 << 11)[:300].astype(np.int64)
    sub = U._graph._CAPI_Slicing(to_dev(selected, dev), 1, _COO, _COO, False)
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    k, o, s = O.row_slice_coo(si, coo, selected)
    _, _, _, row, col = sub._CAPI_COOMetadata()
    assert np.array_equal(row.cpu().numpy(), k) and np.array_equal(col.cpu().numpy(), o)
    assert sub._CAPI_GetNumRows() == 300 and sub._CAPI_GetNumEdges() == k.size


def test_random_walk_and_metapath_flow(dev):
    m, indptr, indices, _ = _rmat_matrix(dev, 11, 15, 6)
    seeds = np.random.default_rng(5).integers(0, 1 << 11, 500).astype(np.int64)
    gs.set_seed(9)
    tr = m.random_walk(to_dev(seeds, dev), 10)
    assert tr.shape == (500, 11)  # memory is [11][500] (reference random_walk.cu:67)
    assert np.array_equal(tr.reshape(-1).cpu().numpy(), O.random_walk(indptr, indices, seeds, 10, seed=9))
    m2, ip2, ix2, _ = _rmat_matrix(dev, 11, 15, 7)
    hm = gs.HeteroMatrix()
    hm.load_from_homo(["a", "b"], [("a", "r0", "b"), ("b", "r1", "a")], [m, m2])
    gs.set_seed(10)
    tr = hm.metapath_random_walk_fused(to_dev(seeds, dev), ["r0", "r1", "r0", "r1"])
    want = O.metapath_walk([indptr, ip2], [indices, ix2], [0, 1, 0, 1], seeds, seed=10)
    assert np.array_equal(tr.reshape(-1).cpu().numpy(), want)
    # the unfused per-step path (hetero_matrix.py:17-24): the -1 of a dead end is fed back in as a
    # column id; it must come back as -1 again, never be dereferenced
    steps = hm.metapath_random_walk(to_dev(seeds, dev), ["r0", "r1", "r0"]).cpu().numpy()
    assert (steps[1] == -1).any()
    graphs = [(indptr, indices), (ip2, ix2), (indptr, indices)]
    for t, (ip, ix) in enumerate(graphs):
        for w in range(500):
            s, d = steps[t, w], steps[t + 1, w]
            assert (d == -1) if s == -1 else (d == -1 or d in ix[ip[s]:ip[s + 1]])


def test_gsddmm_ops(dev):
    m, indptr, indices, _ = _rmat_matrix(dev, 10, 14, 8)
    N, E = 1 << 10, indices.size
    rng = np.random.default_rng(6)
    x = rng.standard_normal((N, 64)).astype(np.float32)
    y = rng.standard_normal((N, 64)).astype(np.float32)
    col = np.repeat(np.arange(N), np.diff(indptr))
    out = gs.ops.u_dot_v(m, to_dev(x, dev), to_dev(y, dev))
    ref = np.einsum("ij,ij->i", x[indices].astype(np.float64), y[col].astype(np.float64))
    scale = np.abs(x[indices] * y[col]).sum(1)
    assert out.shape == (E, 1)
    assert np.all(np.abs(out.cpu().numpy()[:, 0] - ref) <= 1e-5 * scale + 1e-6)
    e = rng.random(E).astype(np.float32) + 0.5
    u = rng.random(N).astype(np.float32) + 0.5
    out = gs.ops.e_div_u(m, to_dev(e, dev), to_dev(u, dev))
    np.testing.assert_allclose(out.cpu().numpy(), e / u[indices], rtol=1e-5)
    out = gs.ops.u_sub_v(m, to_dev(u, dev), to_dev(u, dev), on_format=_CSC)
    np.testing.assert_allclose(out.cpu().numpy(), u[indices] - u[col], rtol=1e-6, atol=1e-7)


def test_errors_are_exceptions_not_aborts(dev):
    A = gs.Graph(False)
    with pytest.raises(RuntimeError, match="not aligned"):
        A._CAPI_LoadCSCWithColIds(torch.arange(3, **I(dev)), torch.arange(3, **I(dev)), torch.arange(2, **I(dev)))
    B = gs.Graph(False)
    B._CAPI_LoadCSC(torch.arange(3), torch.arange(2))  # CPU tensors: the reference LOG(FATAL)s
    with pytest.raises(RuntimeError, match="Not implemented warning"):
        B._CAPI_Slicing(torch.arange(1), 0, _CSC, _CSC, False)
    C, _, _ = graph20(dev)
    with pytest.raises(RuntimeError, match="Not implementation"):
        C._CAPI_Slicing(torch.arange(2, **I(dev)), 0, _CSC, _CSR, False)
    with pytest.raises(RuntimeError, match="No implementation"):
        C._CAPI_Sampling(1, 3, False, _CSC, _CSC)


# ------------------------------------------------ deferred edge count (pending graphs)
def _fused_child(dev, seed=5):
    m, indptr, indices, _ = _rmat_matrix(dev, 12, 16, 9)
    seeds = np.random.default_rng(seed).permutation(1 << 12)[:300].astype(np.int64)
    gs.set_seed(4242)
    sub = m._graph._CAPI_FusedColumnwiseSlicingSampling(to_dev(seeds, dev), 6, False)
    want = O.sample_uniform(indptr, indices, seeds, 6, False, seed=4242, with_coo=False)
    return m, sub, seeds, want


@pytest.mark.parametrize("first_use", ["num_edges", "csc", "sum", "slicing", "coo_rows", "relabel_twice"])
def test_pending_graph_settles_on_first_use(dev, first_use):
    """The fused sampler returns before its edge count has reached the host; whichever method
    touches the graph first must see the finished CSC."""
    m, sub, seeds, (sp, _, rows, _) = _fused_child(dev)
    if first_use == "num_edges":
        assert sub._CAPI_GetNumEdges() == rows.size
    elif first_use == "csc":
        ptr, idx = sub._CAPI_GetCSC()[:2]
        assert np.array_equal(ptr.cpu().numpy(), sp) and np.array_equal(idx.cpu().numpy(), rows)
    elif first_use == "sum":
        s = sub._CAPI_Sum(0, 1, _CSC)
        assert np.array_equal(s.cpu().numpy(), np.diff(sp).astype(np.float32))
    elif first_use == "slicing":
        child = sub._CAPI_Slicing(torch.arange(0, 10, **I(dev)), 0, _CSC, _CSC, False)
        assert child._CAPI_GetNumEdges() == sp[10]
    elif first_use == "coo_rows":
        assert np.array_equal(sub._CAPI_GetCOORows(False).cpu().numpy(), rows)
    else:
        a = sub._CAPI_Relabel()
        b = sub._CAPI_Relabel()  # the second call finds a settled graph
        for x, y in zip(a[:5], b[:5]):
            assert torch.equal(x, y) if torch.is_tensor(x) else x == y
        frontier, (rel,) = O.relabel([seeds, rows], [rows])
        assert np.array_equal(a[0].cpu().numpy(), frontier) and np.array_equal(a[4].cpu().numpy(), rel)
        assert sub._CAPI_GetNumEdges() == rows.size


def test_pending_graph_outlives_its_mailbox_slot(dev):
    """A pending graph kept aside while more calls go by than there are mailbox slots still settles
    (its count is then read from the device)."""
    m, sub, seeds, (sp, _, rows, _) = _fused_child(dev)
    d_seeds = to_dev(seeds, dev)
    for _ in range(80):
        m._graph._CAPI_FusedColumnwiseSlicingSampling(d_seeds[:50], 3, False)._CAPI_Relabel()
    assert sub._CAPI_GetNumEdges() == rows.size
    assert np.array_equal(sub._CAPI_GetCSC()[1].cpu().numpy(), rows)


def test_pending_graph_settled_by_another_thread(dev):
    """A producer thread samples and hands the unsettled graphs over; the consumer (here the
    main thread, after the producer has exited and after calls of its own have used the same
    ticket numbers) relabels them and asks for their edges: it must wait on the producer's
    mailbox slots, not on its own."""
    import threading
    m, indptr, indices, _ = _rmat_matrix(dev, 12, 16, 9)
    rng = np.random.default_rng(11)
    seed_sets = [rng.permutation(1 << 12)[:200 + 40 * i].astype(np.int64) for i in range(4)]
    handed, errors = [], []

    def producer():
        try:
            for i, seeds in enumerate(seed_sets):
                torch.ops.gs_ops._CAPI_SetThreadSeed(600 + i)
                handed.append(m._graph._CAPI_FusedColumnwiseSlicingSampling(to_dev(seeds, dev), 5,
                                                                            False))
        except Exception as e:
            errors.append(e)

    t = threading.Thread(target=producer)
    t.start()
    t.join()
    assert not errors, errors
    # calls of the consumer's own: its ring hands out the ticket numbers the producer's did
    for _ in range(3):
        m._graph._CAPI_FusedColumnwiseSlicingSampling(to_dev(seed_sets[0][:7], dev), 2,
                                                      False)._CAPI_GetNumEdges()
    for i, (sub, seeds) in enumerate(zip(handed, seed_sets)):
        w_ptr, _, w_rows, _ = O.sample_uniform(indptr, indices, seeds, 5, False, seed=600 + i,
                                               with_coo=False)
        if i % 2 == 0:
            frontier, n_src, n_dst, ptr, idx, _, _ = sub._CAPI_Relabel()
            w_frontier, (w_idx,) = O.relabel([seeds, w_rows], [w_rows])
            assert n_dst == seeds.size and n_src == w_frontier.size
            assert np.array_equal(frontier.cpu().numpy(), w_frontier)
            assert np.array_equal(ptr.cpu().numpy(), w_ptr)
            assert np.array_equal(idx.cpu().numpy(), w_idx)
        assert sub._CAPI_GetNumEdges() == w_rows.size
        assert np.array_equal(sub._CAPI_GetCSC()[1].cpu().numpy(), w_rows)


def test_deferred_sampling_switch_gives_identical_results(dev):
    outs = []
    for mode in (True, False):
        torch.ops.gs_ops._CAPI_SetDeferredSampling(mode)
        try:
            _, sub, _, _ = _fused_child(dev, seed=8)
            outs.append(sub._CAPI_Relabel())
        finally:
            torch.ops.gs_ops._CAPI_SetDeferredSampling(True)
    for x, y in zip(outs[0][:5], outs[1][:5]):
        assert torch.equal(x, y) if torch.is_tensor(x) else x == y


def test_unfused_graphsage_flow_with_int32_ids(dev):
    """A graph loaded with int32 ids goes through Slicing -> Sampling -> Relabel (COO <-> CSC
    conversions, sampling over all columns, relabel of both COO sides) and matches the oracle."""
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=2)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, torch.int32))
    seeds = np.random.default_rng(1).permutation(1 << 12)[:200].astype(np.int64)
    sliced = g._CAPI_Slicing(to_dev(seeds, dev, torch.int32), 0, _CSC, _COO, False)
    gs.set_seed(77)
    sampled = sliced._CAPI_Sampling(0, 7, False, _CSC, _COO)
    frontier, n_src, n_dst, row, col, e_ids, fmt = sampled._CAPI_Relabel()
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    sp2, coo2, si2, sel2 = O.sample_uniform(sp, si, None, 7, False, seed=77)
    want_frontier, (rel_col, rel_row) = O.relabel([seeds, si2], [seeds[coo2], si2])
    assert fmt == "coo" and frontier.dtype == torch.int32 and row.dtype == torch.int32
    assert np.array_equal(frontier.cpu().numpy(), want_frontier)
    assert np.array_equal(row.cpu().numpy(), rel_row) and np.array_equal(col.cpu().numpy(), rel_col)
    # CSR of the int32 graph (stable sort on rows) and a row slice on it
    g._CAPI_CSC2CSR()
    r_ip, r_col, r_perm = O.coo2csc(indices, O.csc2coo(indptr, indices.size), 1 << 12, False)
    meta = g._CAPI_Slicing(to_dev(seeds, dev, torch.int32), 1, _CSR, _CSR, False)._CAPI_Metadata()
    w_ip, _, w_col, _ = O.slice_columns(r_ip, r_col, seeds)
    assert np.array_equal(meta[3].cpu().numpy(), w_ip) and np.array_equal(meta[4].cpu().numpy(), w_col)


# ------------------------------------------------------------ super-batch GraphSAGE
def test_super_batch_graphsage_flow_matches_oracle(dev):
    """examples/graphsage/batching.py:59-88: B minibatches sampled as one call, GetBatchCSC,
    BatchCSRRelabel, then the splits; every piece equals what the oracle gives batch by batch."""
    m, indptr, indices, _ = _rmat_matrix(dev, 13, 17, 1)
    g = m._graph
    B, small = 16, 64
    rng = np.random.default_rng(3)
    seeds = np.concatenate([rng.permutation(1 << 13)[:small] for _ in range(B)]).astype(np.int64)
    seeds_ptr = np.arange(B + 1, dtype=np.int64) * small
    d_seeds, d_ptr = to_dev(seeds, dev), to_dev(seeds_ptr, dev)
    for layer, fanout in enumerate([10, 5]):
        gs.set_seed(900 + layer)
        sub = g._CAPI_FusedColumnwiseSlicingSampling(d_seeds, fanout, False)
        ptr, idx, idx_ptr = sub._CAPI_GetBatchCSC(d_ptr)
        uni, uni_ptr, rel, idx_ptr2 = torch.ops.gs_ops.BatchCSRRelabel(d_seeds, d_ptr, idx, idx_ptr)
        sp, _, rows, _ = O.sample_uniform(indptr, indices, seeds, fanout, False, seed=900 + layer,
                                          with_coo=False)
        w_idx_ptr = sp[seeds_ptr]
        w_uni, w_uni_ptr, w_rel = O.batch_csr_relabel(seeds, seeds_ptr, rows, w_idx_ptr)
        assert np.array_equal(ptr.cpu().numpy(), sp) and np.array_equal(idx.cpu().numpy(), rows)
        assert np.array_equal(idx_ptr.cpu().numpy(), w_idx_ptr) and torch.equal(idx_ptr, idx_ptr2)
        assert np.array_equal(uni.cpu().numpy(), w_uni)
        assert np.array_equal(uni_ptr.cpu().numpy(), w_uni_ptr)
        assert np.array_equal(rel.cpu().numpy(), w_rel)
        unit = torch.ops.gs_ops.SplitByOffset(uni, uni_ptr)
        ptrt = torch.ops.gs_ops.IndptrSplitByOffset(ptr, d_ptr)
        indt = torch.ops.gs_ops.SplitByOffset(rel, idx_ptr)
        assert len(unit) == len(ptrt) == len(indt) == B
        for b in range(B):
            lo, hi = seeds_ptr[b], seeds_ptr[b + 1]
            # each piece is the block a separate relabel of that minibatch would give
            f, (r,) = O.relabel([seeds[lo:hi], rows[sp[lo]:sp[hi]]], [rows[sp[lo]:sp[hi]]])
            assert np.array_equal(unit[b].cpu().numpy(), f)
            assert np.array_equal(indt[b].cpu().numpy(), r)
            assert np.array_equal(ptrt[b].cpu().numpy(), sp[lo:hi + 1] - sp[lo])
        seeds, seeds_ptr, d_seeds, d_ptr = w_uni, w_uni_ptr, uni, uni_ptr


def test_indptr_split_by_size(dev):
    indptr = np.concatenate([[0], np.cumsum(np.random.default_rng(0).integers(0, 9, size=103))])
    pieces = torch.ops.gs_ops.IndptrSplitBySize(to_dev(indptr.astype(np.int64), dev), 10)
    assert len(pieces) == 10  # the ragged tail of 3 columns is dropped, as in the reference
    for b, p in enumerate(pieces):
        assert np.array_equal(p.cpu().numpy(), indptr[10 * b:10 * b + 11] - indptr[10 * b])


def test_sampler_threads_on_their_own_streams_are_reproducible(dev):
    """Four host threads, one stream each, run GraphSAGE minibatches at the same time; with a
    seed of its own per minibatch every result equals the oracle's, however they interleave."""
    import threading
    n = 1 << 15
    indptr, indices = rmat_csc_np(n, 1 << 20, seed=41)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, torch.int32))
    rng = np.random.default_rng(7)
    batches = [rng.permutation(n)[:256].astype(np.int64) for _ in range(24)]
    t_batches = [to_dev(b, dev, torch.int32) for b in batches]
    fanouts = (7, 5)
    got = [None] * len(batches)
    errors = []

    def work(k, workers):
        try:
            stream = torch.cuda.Stream(device=dev)
            with torch.cuda.stream(stream):
                for i in range(k, len(batches), workers):
                    torch.ops.gs_ops._CAPI_SetThreadSeed(1000 + i * len(fanouts))
                    seeds, layers = t_batches[i], []
                    for f in fanouts:
                        sub = g._CAPI_FusedColumnwiseSlicingSampling(seeds, f, False)
                        frontier, _, _, ptr, idx, _, _ = sub._CAPI_Relabel()
                        layers.append((ptr, idx, frontier))
                        seeds = frontier
                    stream.synchronize()
                    got[i] = [tuple(t.cpu().numpy().astype(np.int64) for t in l) for l in layers]
        except Exception as e:   # surfaced below: an assert in a thread is otherwise lost
            errors.append(e)

    threads = [threading.Thread(target=work, args=(k, 4)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i, b in enumerate(batches):
        seeds = b
        for l, f in enumerate(fanouts):
            w_ptr, _, w_rows, _ = O.sample_uniform(indptr, indices, seeds, f, False,
                                                   seed=1000 + i * len(fanouts) + l, with_coo=False)
            w_frontier, (w_idx,) = O.relabel([seeds, w_rows], [w_rows])
            ptr, idx, frontier = got[i][l]
            assert np.array_equal(ptr, w_ptr) and np.array_equal(idx, w_idx)
            assert np.array_equal(frontier, w_frontier)
            seeds = w_frontier


@pytest.mark.parametrize("workers", [1, 4])
def test_sample_blocks_pool_equals_the_python_loop(dev, workers):
    """gs.sample_blocks (host threads of the C++ layer, one stream each) against the same
    minibatches sampled one after the other through the Graph methods with the same seeds."""
    m, indptr, indices, _ = _rmat_matrix(dev, 13, 17, 21)
    fanouts = [7, 5, 3]
    rng = np.random.default_rng(8)
    sets = [to_dev(rng.permutation(1 << 13)[:64 + 16 * i].astype(np.int64), dev) for i in range(11)]
    got = gs.sample_blocks(m, sets, fanouts, replace=False, workers=workers, seed=500)
    assert len(got) == len(sets)
    for i, seeds in enumerate(sets):
        torch.ops.gs_ops._CAPI_SetThreadSeed(500 + i * len(fanouts))
        blocks = []
        for k in fanouts:
            sub = m.fused_columnwise_slicing_sampling(seeds, k, False)
            blk = sub.to_dgl_block()
            blocks.insert(0, blk)
            seeds = blk.srcdata["_ID"]
        nodes, got_blocks = got[i]
        assert torch.equal(nodes, seeds)
        for a, b in zip(got_blocks, blocks):
            assert a.num_dst_nodes() == b.num_dst_nodes() and a.num_src_nodes() == b.num_src_nodes()
            assert torch.equal(a.srcdata["_ID"], b.srcdata["_ID"])
            assert torch.equal(a.csc()[0], b.csc()[0]) and torch.equal(a.csc()[1], b.csc()[1])
    gs.set_seed(0)  # back to the shared counter for the tests that follow


_TWO_IN_FLIGHT_OFF = ("switched off in the library: two super-batches in flight passed here and then "
                      "ended a bench run on the weighted 111 M-node graph with a GPU memory fault; the "
                      "likely cause (chained scans of two chip-filling launches starving each other) "
                      "has not been shown on the device")


@pytest.mark.parametrize("workers", [1, pytest.param(2, marks=pytest.mark.skip(reason=_TWO_IN_FLIGHT_OFF)),
                                     pytest.param(3, marks=pytest.mark.skip(reason=_TWO_IN_FLIGHT_OFF))])
def test_sample_blocks_pool_of_super_batches_equals_the_calls_one_by_one(dev, workers):
    """gs.sample_blocks(per_call=...): the seed sets go through the pool as super-batches
    (_CAPI_QueueSampleLayersBatched per group, `workers` groups in flight); every group equals
    the _CAPI_SampleLayersBatched call on it under the group's seed, whatever thread ran it."""
    indptr, indices = rmat_csc_np(1 << 15, 1 << 20, seed=23)
    m = gs.Matrix()
    m.load_csc(to_dev(indptr, dev), to_dev(indices, dev, torch.int32))
    g = m._graph
    fanouts = [15, 10]
    rng = np.random.default_rng(18)
    sets = [to_dev(rng.permutation(1 << 15)[:1024 - 8 * (i % 5)].astype(np.int64), dev, torch.int32)
            for i in range(150)]  # groups of 64, 64 and 22
    per_call = 64
    got = gs.sample_blocks(m, sets, fanouts, workers=workers, seed=300, per_call=per_call)
    assert len(got) == len(sets)
    for grp in range(3):
        part = sets[grp * per_call:(grp + 1) * per_call]
        torch.ops.gs_ops._CAPI_SetThreadSeed(300 + grp * per_call * len(fanouts))
        want = g._CAPI_SampleLayersBatched(part, fanouts, False)
        for b, parts in enumerate(want):
            nodes, blocks = got[grp * per_call + b]
            assert torch.equal(nodes, parts[3])
            assert torch.equal(blocks[0].csc()[1], parts[5]) and torch.equal(blocks[1].csc()[1], parts[2])
            assert torch.equal(blocks[0].csc()[0], parts[4]) and torch.equal(blocks[1].csc()[0], parts[1])
    gs.set_seed(0)
    with pytest.raises(RuntimeError, match="per_call"):
        gs.sample_blocks(m, sets[:2], fanouts, workers=1, per_call=0)
    with pytest.raises(RuntimeError, match="switched off"):
        gs.sample_blocks(m, sets[:2], fanouts, workers=2, per_call=1)
    assert gs.sample_blocks(m, [], fanouts, per_call=4) == []


def test_sample_blocks_rejects_bad_arguments(dev):
    m, _, _, _ = _rmat_matrix(dev, 10, 13, 2)
    seeds = torch.arange(10, device=dev)
    with pytest.raises(RuntimeError, match="workers"):
        gs.sample_blocks(m, [seeds], [3], workers=0)
    with pytest.raises(RuntimeError, match="same GPU"):
        gs.sample_blocks(m, [seeds.cpu()], [3])
    assert gs.sample_blocks(m, [], [3]) == []
    # an error inside a worker comes back as an exception, and the pool goes on working
    with pytest.raises(RuntimeError, match="fanout"):
        gs.sample_blocks(m, [seeds, seeds], [3, -1], workers=2)
    nodes, blocks = gs.sample_blocks(m, [seeds], [3], workers=2)[0]
    assert blocks[0].num_dst_nodes() == 10 and nodes.numel() == blocks[0].num_src_nodes()


def test_relabel_falls_back_when_64_bit_ids_exceed_32_bits(dev):
    """Graph.Relabel behind the fused sampler uses one-word table slots for 64-bit ids; column ids
    beyond 32 bits make it switch to the two-array slots, with the same result as the oracle."""
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=13)
    big = np.int64(1) << 35
    g = gs.Graph(False)
    col_ids = np.arange(1 << 12, dtype=np.int64) + big        # the columns go by huge ids
    g._CAPI_LoadCSCWithColIds(to_dev(col_ids, dev), to_dev(indptr, dev), to_dev(indices, dev))
    seeds = np.random.default_rng(2).permutation(1 << 12)[:300].astype(np.int64)
    for rep in range(2):  # the second call runs on the switched table
        gs.set_seed(90 + rep)
        sub = g._CAPI_FusedColumnwiseSlicingSampling(to_dev(seeds, dev), 6, False)
        frontier, n_src, n_dst, ptr, idx, _, fmt = sub._CAPI_Relabel()
        sp, _, rows, _ = O.sample_uniform(indptr, indices, seeds, 6, False, seed=90 + rep, with_coo=False)
        w_frontier, (w_idx,) = O.relabel([col_ids[seeds], rows], [rows])
        assert np.array_equal(frontier.cpu().numpy(), w_frontier)
        assert np.array_equal(idx.cpu().numpy(), w_idx)
        assert np.array_equal(ptr.cpu().numpy(), sp)
    # ids that fit again keep working on the switched table
    g2 = gs.Graph(False)
    g2._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    gs.set_seed(95)
    sub = g2._CAPI_FusedColumnwiseSlicingSampling(to_dev(seeds, dev), 6, False)
    frontier = sub._CAPI_Relabel()[0]
    sp, _, rows, _ = O.sample_uniform(indptr, indices, seeds, 6, False, seed=95, with_coo=False)
    assert np.array_equal(frontier.cpu().numpy(), O.relabel([seeds, rows], [rows])[0])


# ------------------------------------- a whole minibatch in one call (no host read per layer)
def _oracle_minibatch(indptr, indices, seeds, fanouts, replace, seed, col_ids=None):
    want = []
    cols = seeds
    keys = seeds if col_ids is None else col_ids[seeds]
    for l, k in enumerate(fanouts):
        sp, _, rows, _ = O.sample_uniform(indptr, indices, cols, k, replace, seed=seed + l,
                                          with_coo=False)
        frontier, (renamed,) = O.relabel([keys, rows], [rows])
        want += [frontier, sp, renamed]
        cols = keys = frontier
    return want


def _same(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy().astype(np.int64), w)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("fanouts,replace", [((15, 10, 5), False), ((4, 4), True), ((32,), False),
                                             ((40, 3), False), ((1, 2), True)])
def test_sample_layers_equals_the_layer_loop_and_the_oracle(dev, idt, fanouts, replace):
    """_CAPI_SampleLayers against the oracle run layer by layer and against the Graph methods
    called layer by layer under the same seeds.  Fanouts above 32 without replacement and a
    fanout of 1 with replacement take the loop inside the call."""
    n = 1 << 13
    indptr, indices = rmat_csc_np(n, 1 << 18, seed=17)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, idt))
    seeds = np.random.default_rng(5).permutation(n)[:700].astype(np.int64)
    t_seeds = to_dev(seeds, dev, idt)
    for first in (300, 310):
        gs.set_seed(first)
        got = g._CAPI_SampleLayers(t_seeds, list(fanouts), replace)
        if not (replace and 1 in fanouts):  # (the keep-dim sampler is not the oracle's sample_uniform)
            _same(got, _oracle_minibatch(indptr, indices, seeds, fanouts, replace, first))
        gs.set_seed(first)
        cols, loop = t_seeds, []
        for k in fanouts:
            sub = g._CAPI_FusedColumnwiseSlicingSampling(cols, k, replace)
            r = sub._CAPI_Relabel()
            loop += [r[0], r[3], r[4]]
            cols = r[0]
        for a, b in zip(got, loop):
            assert torch.equal(a, b)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("from_coo", [False, True])
@pytest.mark.parametrize("fanouts,replace", [((15, 10, 5), False), ((4, 4), True), ((40, 3), False)])
def test_sample_layers_on_a_graph_with_edge_data(dev, idt, from_coo, fanouts, replace):
    """A graph with fp32 edge data (configurations 3 and 5 carry weights): the whole
    minibatch still goes in one call, every layer hands back the sampled edges' share of the data
    (`data_[e_ids[select_index]]`, reference src/graph.cc:544-557), and the result equals the
    per-layer calls and the oracle.  Loaded as an unsorted COO the CSC has an edge-id map, and
    the data stays in COO order."""
    n = 1 << 12
    indptr, indices = rmat_csc_np(n, 1 << 17, seed=31)
    rng = np.random.default_rng(9)
    g = gs.Graph(False)
    if from_coo:
        col = np.repeat(np.arange(n, dtype=np.int64), np.diff(indptr))
        perm = rng.permutation(indices.size)
        g._CAPI_LoadCOO(to_dev(indices[perm], dev, idt), to_dev(col[perm], dev, idt))
        g._CAPI_SetMetadata(None, None, n, n)
        g._CAPI_CreateSparseFormat(_CSC)
        t_ptr, t_idx, t_eid = g._CAPI_GetCSC()
        indptr = t_ptr.cpu().numpy()
        indices = t_idx.cpu().numpy().astype(np.int64)
        e_ids = t_eid.cpu().numpy()
        assert not np.array_equal(e_ids, np.arange(e_ids.size))
    else:
        g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, idt))
        e_ids = None
    data = (1.0 - rng.random(indices.size)).astype(np.float32)
    g._CAPI_SetData(to_dev(data, dev))
    seeds = rng.permutation(n)[:600].astype(np.int64)
    t_seeds = to_dev(seeds, dev, idt)
    for first in (410, 420):
        gs.set_seed(first)
        got = g._CAPI_SampleLayers(t_seeds, list(fanouts), replace)
        assert len(got) == 4 * len(fanouts)
        _same([t for i, t in enumerate(got) if i % 4 != 3],
              _oracle_minibatch(indptr, indices, seeds, fanouts, replace, first))
        cols = seeds
        for l, k in enumerate(fanouts):
            sel = O.sample_uniform(indptr, indices, cols, k, replace, seed=first + l,
                                   with_coo=False)[3]
            picked = data[sel] if e_ids is None else data[e_ids[sel]]
            assert np.array_equal(got[4 * l + 3].cpu().numpy(), picked)
            cols = got[4 * l].cpu().numpy().astype(np.int64)
        gs.set_seed(first)
        cols, loop = t_seeds, []
        for k in fanouts:
            sub = g._CAPI_FusedColumnwiseSlicingSampling(cols, k, replace)
            r = sub._CAPI_Relabel()
            loop += [r[0], r[3], r[4], sub._CAPI_GetData("default")]
            cols = r[0]
        for a, b in zip(got, loop):
            assert torch.equal(a, b)
    # the blocks of the Python helper carry the data as edge weights
    gs.set_seed(410)
    _, blocks = gs.sample_layers(g, t_seeds, list(fanouts), replace)
    gs.set_seed(410)
    got = g._CAPI_SampleLayers(t_seeds, list(fanouts), replace)
    assert torch.equal(blocks[-1].edata["w"], got[3])


def test_fused_sampling_settles_its_edge_data_whichever_method_comes_first(dev):
    """The fused sampler hands its child back before the edge count is known; the child's data
    is there whether Relabel, GetData or GetCSC is the first method called on it."""
    n = 1 << 11
    indptr, indices = rmat_csc_np(n, 1 << 15, seed=2)
    data = (1.0 - np.random.default_rng(1).random(indices.size)).astype(np.float32)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    g._CAPI_SetData(to_dev(data, dev))
    seeds = np.arange(0, n, 3, dtype=np.int64)
    sel = O.sample_uniform(indptr, indices, seeds, 5, False, seed=8, with_coo=False)[3]
    for first_call in ("relabel", "data", "csc"):
        gs.set_seed(8)
        sub = g._CAPI_FusedColumnwiseSlicingSampling(to_dev(seeds, dev), 5, False)
        if first_call == "relabel":
            sub._CAPI_Relabel()
        elif first_call == "csc":
            sub._CAPI_GetCSC()
        assert np.array_equal(sub._CAPI_GetData("default").cpu().numpy(), data[sel])
        assert sub._CAPI_GetNumEdges() == sel.size


def test_sample_layers_keeps_8192_seeds_on_the_queued_path(dev):
    """8192 seeds x [15, 10, 5]: bounds of 8.65 M items in the third layer, which the queued chain
    takes (its limit is 2^24 items); the result is the oracle's, and _CAPI_SampleLayersIfQueued
    answers (an empty list would mean the loop)."""
    n = 1 << 17
    indptr, indices = rmat_csc_np(n, 1 << 21, seed=3)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, torch.int32))
    seeds = np.random.default_rng(1).permutation(n)[:8192].astype(np.int64)
    gs.set_seed(90)
    got = g._CAPI_SampleLayersIfQueued(to_dev(seeds, dev, torch.int32), [15, 10, 5], False)
    assert len(got) == 9
    _same(got, _oracle_minibatch(indptr, indices, seeds, (15, 10, 5), False, 90))
    # and one seed more than the bound allows goes layer by layer, with the same result shape
    many = np.random.default_rng(2).permutation(n)[:16000].astype(np.int64)
    assert g._CAPI_SampleLayersIfQueued(to_dev(many, dev, torch.int32), [15, 10, 5], False) == []


@pytest.mark.parametrize("with_data", [False, True])
def test_queued_minibatches_equal_sample_layers_whatever_is_in_flight(dev, with_data):
    """Four minibatches queued before the first is collected, collected out of order: each is
    the minibatch `_CAPI_SampleLayers` gives under the seeds the queue calls took, in call order.
    A graph that cannot be queued (column ids) is sampled at the queue call."""
    m, indptr, indices, data = _rmat_matrix(dev, 13, 17, 21, with_data=with_data)
    g = m._graph
    fanouts = [10, 5, 3]
    sets = [torch.randperm(1 << 13, device=dev)[:300 + 17 * i] for i in range(4)]
    gs.set_seed(400)
    want = [g._CAPI_SampleLayers(s, fanouts, False) for s in sets]
    gs.set_seed(400)
    handles = [g._CAPI_QueueSampleLayers(s, fanouts, False) for s in sets]
    for i in (2, 0, 3, 1):
        got = handles[i].collect()
        assert len(got) == len(want[i]) == (4 if with_data else 3) * len(fanouts)
        for a, b in zip(got, want[i]):
            assert torch.equal(a, b)
    with pytest.raises(RuntimeError, match="collected already"):
        handles[0].collect()
    # the Python helper returns blocks
    gs.set_seed(400)
    nodes, blocks = gs.queue_sample_layers(m, sets[0], fanouts).collect()
    assert torch.equal(nodes, want[0][-(4 if with_data else 3)]) and len(blocks) == 3
    # a graph with column ids is sampled layer by layer at the queue call
    col_ids = to_dev(np.random.default_rng(1).permutation(1 << 13).astype(np.int64), dev)
    sub = gs.Graph(False)
    sub._CAPI_LoadCSCWithColIds(col_ids, to_dev(indptr, dev), to_dev(indices, dev))
    seeds = torch.arange(100, device=dev)
    gs.set_seed(77)
    loop = sub._CAPI_SampleLayers(seeds, [4], False)
    gs.set_seed(77)
    for a, b in zip(sub._CAPI_QueueSampleLayers(seeds, [4], False).collect(), loop):
        assert torch.equal(a, b)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_sample_layers_with_no_seeds_and_with_isolated_seeds(dev, idt):
    """No seeds at all, and seeds without neighbours (every later layer is then empty too):
    lengths 0 all the way, offsets of the right length, no launch goes wrong."""
    indptr = np.array([0, 0, 2, 2, 3], dtype=np.int64)   # columns 0 and 2 have no edges
    indices = np.array([3, 1, 1], dtype=np.int64)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, idt))
    for seeds in (np.zeros(0, dtype=np.int64), np.array([0, 2], dtype=np.int64),
                  np.array([1, 3, 0], dtype=np.int64)):
        gs.set_seed(3)
        got = g._CAPI_SampleLayers(to_dev(seeds, dev, idt), [2, 2, 2], False)
        _same(got, _oracle_minibatch(indptr, indices, seeds, (2, 2, 2), False, 3))


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("fanout,replace", [(2, False), (2, True), (1, True), (40, False)])
def test_sampling_a_slice_without_edges(dev, idt, fanout, replace):
    """Slice first, then sample (the sampler without the fused operator): when none of the
    seeds has a neighbour the slice holds no edge at all, and every kind of column sampling
    of it is an empty graph over the same columns."""
    indptr = np.array([0, 0, 2, 2, 3], dtype=np.int64)   # columns 0 and 2 have no edges
    indices = np.array([3, 1, 1], dtype=np.int64)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, idt))
    sliced = g._CAPI_Slicing(to_dev(np.array([0, 2, 0], dtype=np.int64), dev, idt), 0, _CSC, _COO,
                             False)
    assert sliced._CAPI_GetNumEdges() == 0
    probs = torch.zeros(0, **F(dev))
    for sub in (sliced._CAPI_Sampling(0, fanout, replace, _CSC, _COO),
                sliced._CAPI_Sampling(0, fanout, replace, _CSC, _CSC),
                sliced._CAPI_SamplingWithProbs(0, probs, min(fanout, 32), replace, _CSC, _COO)):
        ptr, idx, _ = sub._CAPI_GetCSC()
        if fanout == 1 and replace and idx.numel():  # one slot per column, -1 where it is empty
            assert idx.cpu().tolist() == [-1, -1, -1] and ptr.cpu().tolist() == [0, 1, 2, 3]
            continue
        assert ptr.cpu().tolist() == [0, 0, 0, 0] and idx.numel() == 0
        frontier = sub._CAPI_Relabel()[0]
        assert frontier.cpu().tolist() == [0, 2]


def test_sample_layers_python_helper_returns_blocks(dev):
    m, indptr, indices, _ = _rmat_matrix(dev, 12, 16, 3)
    seeds = to_dev(np.arange(100, dtype=np.int64), dev)
    gs.set_seed(5)
    nodes, blocks = gs.sample_layers(m, seeds, [4, 3])
    gs.set_seed(5)
    want = _oracle_minibatch(indptr, indices, np.arange(100, dtype=np.int64), (4, 3), False, 5)
    assert np.array_equal(nodes.cpu().numpy(), want[3])
    assert [b.num_dst_nodes() for b in blocks] == [want[0].size, 100]
    assert np.array_equal(blocks[1].csc()[1].cpu().numpy(), want[2])


def test_sample_layers_on_a_graph_with_column_ids_takes_the_loop(dev):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=13)
    col_ids = np.random.default_rng(1).permutation(1 << 12).astype(np.int64)
    g = gs.Graph(False)
    g._CAPI_LoadCSCWithColIds(to_dev(col_ids, dev), to_dev(indptr, dev), to_dev(indices, dev))
    seeds = np.arange(200, dtype=np.int64)
    gs.set_seed(77)
    got = g._CAPI_SampleLayers(to_dev(seeds, dev), [5], False)
    _same(got, _oracle_minibatch(indptr, indices, seeds, (5,), False, 77, col_ids=col_ids))


def test_sample_layers_repeats_layer_by_layer_when_an_id_exceeds_32_bits(dev):
    """The queued layers keep 64-bit ids on one-word table slots.  A neighbour id beyond 32 bits
    is reported by the kernels, the minibatch is sampled again layer by layer under the same
    seeds, and the calling thread stays on that path.  (Run in a thread of its own: the switch is
    per thread.)"""
    import threading
    indptr = np.array([0, 2, 4, 6, 6], dtype=np.int64)
    indices = np.array([1, 2, 0, (1 << 33) + 5, 0, 1], dtype=np.int64)
    seeds = np.array([0, 1, 2], dtype=np.int64)
    failure = []

    def body():
        try:
            torch.cuda.set_device(dev)
            g = gs.Graph(False)
            g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
            for first in (11, 12):
                torch.ops.gs_ops._CAPI_SetThreadSeed(first)
                got = g._CAPI_SampleLayers(to_dev(seeds, dev), [2, 2], False)
                _same(got, _oracle_minibatch(indptr, indices, seeds, (2, 2), False, first))
        except BaseException as e:  # noqa: BLE001
            failure.append(e)

    t = threading.Thread(target=body)
    t.start()
    t.join()
    if failure:
        raise failure[0]


@pytest.mark.parametrize("whole_minibatch", [True, False])
def test_a_look_back_that_gave_up_is_reported_and_does_not_stick(dev, whole_minibatch):
    """The error word a tile raises when its bounded wait runs out stays in the look-back state.
    Raised here from the host (every kernel runs to its end): the call that meets it fails with an
    exception, the host layer clears the state behind it, and the next call is right again."""
    n = 1 << 12
    indptr, indices = rmat_csc_np(n, 1 << 16, seed=4)
    g = gs.Graph(False)
    t_ptr = to_dev(indptr, dev)
    g._CAPI_LoadCSC(t_ptr, to_dev(indices, dev, torch.int32))
    seeds = np.random.default_rng(0).permutation(n)[:500].astype(np.int64)
    t_seeds = to_dev(seeds, dev, torch.int32)

    def run(first):
        gs.set_seed(first)
        if whole_minibatch:
            return g._CAPI_SampleLayers(t_seeds, [6, 4], False)
        out, cols = [], t_seeds
        for k in (6, 4):
            r = g._CAPI_FusedColumnwiseSlicingSampling(cols, k, False)._CAPI_Relabel()
            out += [r[0], r[3], r[4]]
            cols = r[0]
        return out

    _same(run(20), _oracle_minibatch(indptr, indices, seeds, (6, 4), False, 20))
    torch.ops.gs_ops._CAPI_DebugRaiseLookbackError(t_ptr)
    with pytest.raises(RuntimeError, match="gave up"):
        run(21)
    for first in (22, 23):
        _same(run(first), _oracle_minibatch(indptr, indices, seeds, (6, 4), False, first))
