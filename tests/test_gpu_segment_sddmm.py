"""GPU parity: segment sums / normalise / EDivUSum and SDDMM vs the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import graph_12col_4edge, graph_20x5, rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu
RTOL = 1e-5  # float values: relative tolerance of the parity contract
ID_DTYPES = [torch.int64, torch.int32]


def _seg_sum(dev, indptr, data, powk, e_ids=None, n_ids=None, out_size=None, idt=torch.int64):
    out_size = out_size or indptr.size - 1
    out = torch.zeros(out_size, dtype=torch.float32, device=dev)
    capi.segment_sum(to_dev(indptr, dev), None if e_ids is None else to_dev(e_ids, dev),
                     None if n_ids is None else to_dev(n_ids, dev, idt), to_dev(data, dev), powk, out)
    return out.cpu().numpy()


def test_sum_reference_vectors(dev):
    # reference tests/test_graph_compute.cc:8-74
    indptr, _ = graph_20x5()
    ones = np.ones(100, dtype=np.float32)
    assert np.array_equal(_seg_sum(dev, indptr, ones, 1), np.full(20, 5, np.float32))
    assert np.array_equal(_seg_sum(dev, indptr, ones, 2), np.full(20, 5, np.float32))
    data = np.tile(np.arange(1, 6, dtype=np.float32), 20)
    assert np.array_equal(_seg_sum(dev, indptr, data, 1), np.full(20, 15, np.float32))
    assert np.array_equal(_seg_sum(dev, indptr, data, 2), np.full(20, 55, np.float32))


def test_row_sum_reference_vector_coo(dev):
    # reference tests/test_graph_compute.cc:93-108: rows 1 and 3 of the 12-column graph
    indptr, indices = graph_12col_4edge()
    data = np.arange(3, 7, dtype=np.float32)
    out = torch.zeros(12, dtype=torch.float32, device=dev)
    capi.coo_sum(to_dev(indices, dev), None, to_dev(data, dev), 1, out)
    expected = np.array([0, 8, 0, 10] + [0] * 8, dtype=np.float32)
    assert np.array_equal(out.cpu().numpy(), expected)
    assert np.array_equal(O.coo_sum(indices, None, data, 1, 12), expected)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("powk", [1, 2, 3])
@pytest.mark.parametrize("maps", [False, True])
def test_segment_sum_rmat(dev, powk, maps, idt):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=4)  # hubs of several thousand edges
    rng = np.random.default_rng(powk)
    data = rng.random(indices.size, dtype=np.float32)
    e_ids = rng.permutation(indices.size).astype(np.int64) if maps else None
    n_ids = rng.permutation(indptr.size - 1).astype(np.int64) if maps else None
    got = _seg_sum(dev, indptr, data, powk, e_ids, n_ids, idt=idt)
    want = O.segment_sum(indptr, e_ids, n_ids, data, powk, indptr.size - 1)
    np.testing.assert_allclose(got, want, rtol=RTOL)
    short = np.diff(indptr) <= 16  # short segments are summed in edge order: bit exact
    idx = np.arange(indptr.size - 1) if n_ids is None else n_ids
    assert np.array_equal(got[idx[short]], want[idx[short]])


@pytest.mark.parametrize("case", ["hub_over_chunks", "chunk_aligned", "empties_then_long",
                                  "one_segment", "short_over_chunk_border", "few_edges_into_next_chunk"])
@pytest.mark.parametrize("maps", [False, True])
def test_segment_sum_pieces_across_chunks(dev, case, maps):
    # long segments are summed by chunks of 1024 edges of the edge array: segments that start,
    # cover and end chunks, with short and empty segments around them
    rng = np.random.default_rng(7)
    deg = {
        "hub_over_chunks": [3, 0, 5000, 2, 17, 0, 0, 1030, 16, 2500, 1],
        "chunk_aligned": [1024, 2048, 1024, 0, 1024],
        "empties_then_long": [0] * 3000 + [40] + [0] * 2000 + [3000] + [0] * 100,
        "one_segment": [10000],
        "short_over_chunk_border": [1020, 8, 1020, 16, 17, 2000],
        # long segments of which 1, 19 and 3 edges reach into the next chunk, and one that starts
        # one edge before a border
        "few_edges_into_next_chunk": [1007, 18, 3, 1019, 20, 17, 991, 40],
    }[case]
    indptr = np.concatenate([[0], np.cumsum(np.asarray(deg, dtype=np.int64))])
    nnz, n = int(indptr[-1]), len(deg)
    data = rng.random(nnz, dtype=np.float32)
    e_ids = rng.permutation(nnz).astype(np.int64) if maps else None
    n_ids = rng.permutation(n).astype(np.int64) if maps else None
    got = _seg_sum(dev, indptr, data, 2, e_ids, n_ids)
    src = data if e_ids is None else data[e_ids]
    want = np.zeros(n)
    for s in range(n):  # float64: the order of the additions is not the sequential one
        want[s if n_ids is None else n_ids[s]] = np.sum(src[indptr[s]:indptr[s + 1]].astype(np.float64) ** 2)
    np.testing.assert_allclose(got, want, rtol=RTOL)
    assert np.array_equal(got, _seg_sum(dev, indptr, data, 2, e_ids, n_ids))  # fixed order
    # normalize over the same layout
    out = torch.empty(nnz, dtype=torch.float32, device=dev)
    capi.segment_normalize(to_dev(indptr, dev), None if e_ids is None else to_dev(e_ids, dev),
                           to_dev(data + 0.1, dev), out)
    src = (data + 0.1) if e_ids is None else (data + 0.1)[e_ids]
    want_n = np.empty(nnz)
    for s in range(n):
        seg = src[indptr[s]:indptr[s + 1]].astype(np.float64)
        pos = np.arange(indptr[s], indptr[s + 1]) if e_ids is None else e_ids[indptr[s]:indptr[s + 1]]
        want_n[pos] = seg / seg.sum()
    np.testing.assert_allclose(out.cpu().numpy(), want_n, rtol=RTOL)


@pytest.mark.parametrize("seed", range(12))
def test_segment_sum_random_layouts(dev, seed):
    # random mixes of empty, short, just-long and multi-chunk segments: wherever the chunk borders
    # fall, sums and normalised weights agree with float64
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(1, 600))
    deg = rng.choice([0, 1, 5, 16, 17, 18, 30, 100, 1030, 2500, 3], size=n,
                     p=[.2, .1, .1, .1, .1, .1, .1, .1, .03, .02, .05])
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    nnz = int(indptr[-1])
    data = (rng.random(nnz, dtype=np.float32) + np.float32(0.05))
    got = _seg_sum(dev, indptr, data, 1)
    want = np.array([data[indptr[s]:indptr[s + 1]].astype(np.float64).sum() for s in range(n)])
    np.testing.assert_allclose(got, want, rtol=RTOL)
    if nnz:
        out = torch.empty(nnz, dtype=torch.float32, device=dev)
        capi.segment_normalize(to_dev(indptr, dev), None, to_dev(data, dev), out)
        want_n = data.astype(np.float64) / np.repeat(want, deg)
        np.testing.assert_allclose(out.cpu().numpy(), want_n, rtol=RTOL)


@pytest.mark.parametrize("shift", [0, 1, 3])
def test_segment_sum_hubs_and_unaligned_data(dev, shift):
    # segments of many whole 1024-edge chunks (summed without marks), their partial chunks at
    # both ends shared with short and just-long neighbours, and weights that start 4 or 12 bytes
    # off a 16-byte boundary (the by-edge pass then reads edge by edge instead of four at a time)
    rng = np.random.default_rng(shift)
    deg = np.array([3, 5000, 17, 0, 20000, 1, 1024, 1024, 40, 3 * 1024 + 1, 16, 70000, 2],
                   dtype=np.int64)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    nnz = int(indptr[-1])
    data = (rng.random(nnz, dtype=np.float32) + np.float32(0.05))
    base = torch.empty(nnz + 8, dtype=torch.float32, device=dev)
    d_data = base[shift:shift + nnz]
    d_data.copy_(to_dev(data, dev))
    out_base = torch.empty(nnz + 8, dtype=torch.float32, device=dev)
    for powk in (1, 2):
        got = torch.empty(deg.size, dtype=torch.float32, device=dev)
        capi.segment_sum(to_dev(indptr, dev), None, None, d_data, powk, got)
        want = np.array([(data[indptr[s]:indptr[s + 1]].astype(np.float64) ** powk).sum()
                         for s in range(deg.size)])
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=RTOL)
    want = np.array([data[indptr[s]:indptr[s + 1]].astype(np.float64).sum() for s in range(deg.size)])
    out = out_base[shift:shift + nnz]
    capi.segment_normalize(to_dev(indptr, dev), None, d_data, out)
    np.testing.assert_allclose(out.cpu().numpy(), data.astype(np.float64) / np.repeat(want, deg),
                               rtol=RTOL)
    # through an edge map: weights stored in another order
    perm = rng.permutation(nnz).astype(np.int64)
    stored = np.empty_like(data)
    stored[perm] = data
    got = torch.empty(deg.size, dtype=torch.float32, device=dev)
    capi.segment_sum(to_dev(indptr, dev), to_dev(perm, dev), None, to_dev(stored, dev), 1, got)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=RTOL)


def test_segment_sum_edge_count_is_an_upper_bound(dev):
    # the data array may be longer than the offsets cover: the rest is not read into any sum
    indptr = np.array([0, 2000, 2003], dtype=np.int64)
    data = np.ones(5000, dtype=np.float32)
    assert np.array_equal(_seg_sum(dev, indptr, data, 1), np.array([2000, 3], np.float32))


def test_segment_sum_mostly_empty(dev):
    # the layer-wise sampler case: one segment per graph row, almost all empty
    n = 300000
    rng = np.random.default_rng(0)
    deg = np.zeros(n, dtype=np.int64)
    deg[rng.integers(0, n, 4000)] = rng.integers(1, 17, 4000)  # <= 16 edges: summed in edge order
    indptr = np.concatenate([[0], np.cumsum(deg)])
    data = rng.random(int(indptr[-1]), dtype=np.float32)
    got = _seg_sum(dev, indptr, data, 2)
    assert np.array_equal(got, O.segment_sum(indptr, None, None, data, 2, n))


@pytest.mark.parametrize("maps", [False, True])
def test_segment_normalize(dev, maps):
    indptr, indices = rmat_csc_np(1 << 11, 1 << 16, seed=5)
    rng = np.random.default_rng(1)
    data = rng.random(indices.size, dtype=np.float32) + 0.1
    e_ids = rng.permutation(indices.size).astype(np.int64) if maps else None
    out = torch.empty(indices.size, dtype=torch.float32, device=dev)
    capi.segment_normalize(to_dev(indptr, dev), None if e_ids is None else to_dev(e_ids, dev),
                           to_dev(data, dev), out)
    want = O.segment_normalize(indptr, e_ids, data)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=RTOL)
    # every non-empty segment sums to 1
    got = out.cpu().numpy()
    d = got if e_ids is None else got[e_ids]
    sums = np.add.reduceat(np.concatenate([d, [0]]), indptr[:-1])[np.diff(indptr) > 0]
    np.testing.assert_allclose(sums, 1.0, rtol=1e-4)


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_coo_sum_and_e_div_u_sum(dev, idt):
    indptr, indices = rmat_csc_np(1 << 11, 1 << 16, seed=6)
    col = O.csc2coo(indptr, indices.size)
    rng = np.random.default_rng(2)
    data = rng.random(indices.size, dtype=np.float32)
    out = torch.zeros(1 << 11, dtype=torch.float32, device=dev)
    capi.coo_sum(to_dev(indices, dev, idt), None, to_dev(data, dev), 2, out)
    np.testing.assert_allclose(out.cpu().numpy(), O.coo_sum(indices, None, data, 2, 1 << 11), rtol=1e-4)
    divisor = rng.random(1 << 11, dtype=np.float32) + 0.5
    od = torch.zeros(indices.size, dtype=torch.float32, device=dev)
    osum = torch.zeros(1 << 11, dtype=torch.float32, device=dev)
    capi.e_div_u_sum(to_dev(indices, dev, idt), to_dev(col, dev, idt), to_dev(data, dev),
                     to_dev(divisor, dev), od, osum)
    wd, ws = O.e_div_u_sum(indices, col, data, divisor, 1 << 11)
    assert np.array_equal(od.cpu().numpy(), wd)  # one IEEE division per edge: bit exact
    np.testing.assert_allclose(osum.cpu().numpy(), ws, rtol=1e-4)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("targets,edges,skew", [
    (2_450_000, 1 << 20, True),    # a LADIES row sum: many targets, hubs among them
    (2_450_000, 1 << 20, False),
    (1000, 1 << 18, False),        # fewer targets than runs: every run is one target
    (1 << 23, 300_000, True),      # the widest runs (2^15 sums in LDS)
    ((1 << 23) + 1, 300_000, False),  # one target too many for the runs: the plain kernel
    (70_000, (1 << 17) - 1, False),   # one edge short of the binned path
    (5, 1 << 19, False),           # one run shared by several workgroups
])
def test_coo_sum_binned(dev, idt, targets, edges, skew):
    """The sums with a known number of targets: against float64 sums of the same products (the
    order of the additions is not fixed, so a tolerance), on top of what `out` held, for sizes
    on both sides of every switch between the binned and the plain kernel."""
    rng = np.random.default_rng(edges + targets)
    if skew:
        t = (rng.random(edges) ** 6 * targets).astype(np.int64)  # most edges on a few low targets
    else:
        t = rng.integers(0, targets, size=edges)
    t[:3] = [0, targets - 1, targets - 1]
    data = (rng.random(edges, dtype=np.float32) + 0.25).astype(np.float32)
    for powk in (1, 2):
        before = rng.random(targets, dtype=np.float32)
        out = to_dev(before, dev)
        capi.coo_sum_binned(to_dev(t, dev, idt), None, to_dev(data, dev), powk, out)
        want = before.astype(np.float64) + np.bincount(t, weights=data.astype(np.float64) ** powk,
                                                       minlength=targets)
        np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-5)
        # targets nobody hits keep exactly what they held
        idle = np.bincount(t, minlength=targets) == 0
        assert np.array_equal(out.cpu().numpy()[idle], before[idle])
    # with an edge-id map the plain kernel takes the call, whatever the size
    e_ids = rng.permutation(edges)
    out = torch.zeros(targets, dtype=torch.float32, device=dev)
    capi.coo_sum_binned(to_dev(t, dev, idt), to_dev(e_ids, dev), to_dev(data, dev), 1, out)
    want = np.bincount(t, weights=data[e_ids].astype(np.float64), minlength=targets)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-5)


@pytest.mark.parametrize("edges", [1 << 18, 5000])
def test_coo_sum_binned_leaves_out_targets_beyond_the_output(dev, edges):
    """A target outside [0, num_targets) is left out on the binned path (2^18 edges) and on the
    plain kernel the smaller call is passed on to; the slots behind `out` stay untouched."""
    targets = 1000
    rng = np.random.default_rng(edges)
    t = rng.integers(0, targets + 200, size=edges)
    t[:4] = [-1, -5, targets, 1 << 30]
    data = (rng.random(edges, dtype=np.float32) + 0.25).astype(np.float32)
    buf = torch.full((targets + 4096,), 7.0, dtype=torch.float32, device=dev)
    out = buf[:targets]
    out.zero_()
    capi.coo_sum_binned(to_dev(t, dev, torch.int32), None, to_dev(data, dev), 1, out)
    ok = (t >= 0) & (t < targets)
    want = np.bincount(t[ok], weights=data[ok].astype(np.float64), minlength=targets)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-5)
    assert bool((buf[targets:] == 7.0).all())


# ------------------------------------------------------------------ SDDMM
def _sddmm_coo_gpu(dev, op, row, col, e_ids, lhs, rhs, lt, rt, idt=torch.int64):
    ls = lhs.shape if lhs.ndim > 1 else lhs.shape + (1,)
    rs = rhs.shape if rhs.ndim > 1 else rhs.shape + (1,)
    b = O.calc_bcast(op, ls, rs)
    out = torch.zeros((row.size, b["out_len"]), dtype=torch.float32, device=dev)
    capi.sddmm_coo(op, to_dev(row, dev, idt), to_dev(col, dev, idt),
                   None if e_ids is None else to_dev(e_ids, dev),
                   to_dev(lhs, dev), to_dev(rhs, dev), out, lt, rt, b["lhs_len"], b["rhs_len"],
                   b["out_len"], b["reduce_size"],
                   None if b["lhs_off"] is None else to_dev(b["lhs_off"], dev),
                   None if b["rhs_off"] is None else to_dev(b["rhs_off"], dev))
    return out.cpu().numpy()


def test_sddmm_reference_vectors(dev):
    # reference tests/test_sddmm.cc:7-36 (u_add_v on COO) and :95-107 (on CSC)
    r = np.arange(100, dtype=np.int64)
    f = np.arange(100, dtype=np.float32)
    got = _sddmm_coo_gpu(dev, "add", r, r, None, f, f, 0, 2)
    assert np.array_equal(got[:, 0], f * 2)
    indptr, indices = graph_20x5()
    rhs = np.arange(20, dtype=np.float32)
    out = torch.zeros((100, 1), dtype=torch.float32, device=dev)
    capi.sddmm_csc("add", to_dev(indptr, dev), to_dev(indices, dev), None, None, to_dev(f, dev),
                   to_dev(rhs, dev), out, 0, 2, 1, 1, 1, 1)
    assert np.array_equal(out.cpu().numpy()[:, 0], f + np.repeat(rhs, 5))


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "copy_lhs", "copy_rhs", "dot"])
@pytest.mark.parametrize("targets", [(0, 2), (2, 0), (1, 2), (0, 1)])
def test_sddmm_coo_ops_targets(dev, op, targets):
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=7)
    col = O.csc2coo(indptr, indices.size)
    E, N = indices.size, 1 << 10
    rng = np.random.default_rng(3)
    lt, rt = targets
    lhs = rng.random((E if lt == 1 else N, 8), dtype=np.float32) + 0.5
    rhs = rng.random((E if rt == 1 else N, 8), dtype=np.float32) + 0.5
    e_ids = rng.permutation(E).astype(np.int64)
    got = _sddmm_coo_gpu(dev, op, indices, col, e_ids, lhs, rhs, lt, rt)
    want = O.sddmm_coo(op, indices, col, e_ids, lhs, rhs, lt, rt)
    if op == "dot":
        np.testing.assert_allclose(got, want, rtol=RTOL)
    else:
        assert np.array_equal(got, want)
    # closed form (dense gather)
    sel = {0: indices, 1: e_ids, 2: col}
    L, R = lhs[sel[lt]], rhs[sel[rt]]
    dense = {"add": L + R, "sub": L - R, "mul": L * R, "div": L / R, "copy_lhs": L, "copy_rhs": R,
             "dot": (L * R).sum(1, keepdims=True)}[op]
    full = np.zeros_like(want)
    full[e_ids] = dense
    np.testing.assert_allclose(want, full, rtol=RTOL)


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_sddmm_dot_64_fast_path(dev, idt):
    # u_dot_v with 64-wide fp32 features (the large-graph configuration of the benchmark)
    indptr, indices = rmat_csc_np(1 << 11, 1 << 16, seed=8)
    col = O.csc2coo(indptr, indices.size)
    rng = np.random.default_rng(4)
    lhs = rng.standard_normal((1 << 11, 64)).astype(np.float32)
    rhs = rng.standard_normal((1 << 11, 64)).astype(np.float32)
    got = _sddmm_coo_gpu(dev, "dot", indices, col, None, lhs, rhs, 0, 2, idt=idt)
    want = O.sddmm_coo("dot", indices, col, None, lhs, rhs, 0, 2)
    ref = np.einsum("ij,ij->i", lhs[indices].astype(np.float64), rhs[col].astype(np.float64))
    scale = np.abs(lhs[indices] * rhs[col]).sum(1)  # error bound relative to the summed magnitudes
    assert np.all(np.abs(got[:, 0] - ref) <= RTOL * scale + 1e-6)
    assert np.all(np.abs(want[:, 0] - ref) <= RTOL * scale + 1e-6)


def test_sddmm_broadcast(dev):
    # worked example of the reference (src/bcast.h:20-30): lhs (1,3) op rhs (5,1) -> (5,3)
    b = O.calc_bcast("add", (7, 1, 3), (7, 5, 1))
    assert b["lhs_off"].tolist() == [0, 1, 2] * 5
    assert b["rhs_off"].tolist() == [i for i in range(5) for _ in range(3)]
    indptr, indices = rmat_csc_np(1 << 8, 1 << 11, seed=9)
    col = O.csc2coo(indptr, indices.size)
    rng = np.random.default_rng(5)
    lhs = rng.random((1 << 8, 1, 3), dtype=np.float32)
    rhs = rng.random((1 << 8, 5, 1), dtype=np.float32)
    got = _sddmm_coo_gpu(dev, "mul", indices, col, None, lhs, rhs, 0, 2)
    want = (lhs[indices] * rhs[col]).reshape(indices.size, 15)
    assert np.array_equal(got, want)
    assert np.array_equal(O.sddmm_coo("mul", indices, col, None, lhs, rhs, 0, 2), want)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("use_maps", [False, True])
def test_sddmm_csc(dev, use_maps, idt):
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=10)
    E, N = indices.size, 1 << 10
    rng = np.random.default_rng(6)
    lhs = rng.random((N, 4), dtype=np.float32)
    rhs = rng.random((2 * N, 4), dtype=np.float32)
    e_ids = rng.permutation(E).astype(np.int64) if use_maps else None
    nid = (rng.permutation(N) + N).astype(np.int64) if use_maps else None
    out = torch.zeros((E, 4), dtype=torch.float32, device=dev)
    capi.sddmm_csc("add", to_dev(indptr, dev), to_dev(indices, dev, idt),
                   None if e_ids is None else to_dev(e_ids, dev),
                   None if nid is None else to_dev(nid, dev, idt),
                   to_dev(lhs, dev), to_dev(rhs, dev), out, 0, 2, 4, 4, 4, 1)
    want = O.sddmm_csc("add", indptr, indices, e_ids, nid, lhs, rhs, 0, 2)
    assert np.array_equal(out.cpu().numpy(), want)
