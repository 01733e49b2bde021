"""GPU: the tail of a layer-wise sampler (node set, kept rows of a column slice, block values)
through the C ABI against numpy, and the one-call layer against the operator chain it stands
for (examples/ladies/ladies_raw.py:10-25)."""
import numpy as np
import pytest
import torch

import graph_sampling_amd as gs
from graph_sampling_amd import capi
from graph_sampling_amd.format import _COO, _CSC, _CSR
from graph_sampling_amd.jit import passes
from oracle import oracle as O
from tests.util import rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu

IDT = {4: (np.int32, torch.int32), 8: (np.int64, torch.int64)}


@pytest.mark.parametrize("idb", [4, 8])
@pytest.mark.parametrize("na,nb", [(1, 0), (0, 1), (5, 3), (512, 512), (1000, 24), (3000, 1096)])
def test_sorted_union_is_numpy_unique(dev, idb, na, nb):
    npt, _ = IDT[idb]
    rng = np.random.default_rng(na * 7 + nb)
    # a narrow range, so that values repeat inside and across the two lists
    a = rng.integers(0, max(2, (na + nb) // 2), na).astype(npt)
    b = rng.integers(0, max(2, (na + nb) // 2), nb).astype(npt)
    out, count = capi.sorted_union(to_dev(a, dev), to_dev(b, dev))
    want = np.unique(np.concatenate([a, b]))
    n = int(count.item())
    assert n == want.size
    assert np.array_equal(out[:n].cpu().numpy(), want)


def test_sorted_union_at_its_limit_and_beyond(dev):
    for idb, (npt, _) in IDT.items():
        most = capi.sorted_union_max(idb)
        ids = np.random.default_rng(idb).permutation(10 * most)[:most].astype(npt)
        ids[-1] = np.iinfo(npt).max - 1  # large ids sort last, not as padding
        out, count = capi.sorted_union(to_dev(ids[:most // 2], dev), to_dev(ids[most // 2:], dev))
        assert int(count.item()) == most
        assert np.array_equal(out.cpu().numpy(), np.sort(ids))
        with pytest.raises(capi.GsError):
            capi.sorted_union(to_dev(ids, dev), to_dev(ids[:1], dev))


def _np_pick(row, col, nodes, bits):
    place = np.searchsorted(nodes, row)
    place[place >= nodes.size] = 0
    keep = nodes[place] == row
    pos = np.nonzero(keep)[0]
    return (col[pos].astype(np.int64) << bits) | place[pos], pos


@pytest.mark.parametrize("idb", [4, 8])
@pytest.mark.parametrize("E,num_nodes,room", [(1, 1, 1), (5000, 40, 64), (100_000, 700, 1024),
                                              (300_001, 1500, 4096), (1_000_000, 4000, 4096),
                                              (20_000, 4000, 4096)])
def test_pick_rows_and_block_values_against_numpy(dev, idb, E, num_nodes, room):
    npt, tt = IDT[idb]
    rng = np.random.default_rng(E)
    # (20 000 edges over two columns: more edges in a column than its workgroup holds in LDS)
    N, S = 5000, (2 if E == 20_000 else 300)
    row = rng.integers(0, N, E).astype(npt)
    col = np.sort(rng.integers(0, S, E)).astype(npt)
    nodes = np.sort(rng.permutation(N)[:num_nodes]).astype(npt)
    padded = np.concatenate([nodes, np.full(room - num_nodes, -7, npt)])  # beyond the count: unread
    count = torch.tensor([num_nodes], dtype=torch.int64, device=dev)
    key, pos, totals = capi.coo_pick_rows(to_dev(row, dev), to_dev(col, dev), to_dev(padded, dev),
                                          count, room)
    bits = int(np.ceil(np.log2(room))) if room > 1 else 0
    want_key, want_pos = _np_pick(row, col, nodes, bits)
    got_n, kept = [int(x) for x in totals.cpu()]
    assert got_n == num_nodes and kept == want_pos.size
    # the same count through a mailbox, and any device value through gs_post_total
    box = capi.Mailbox()
    assert capi.coo_pick_rows(to_dev(row, dev), to_dev(col, dev), to_dev(padded, dev), count, room,
                              box)[3] == kept
    assert capi.post_total(totals, 0, box) == num_nodes and capi.post_total(totals, 1, box) == kept
    assert np.array_equal(key[:kept].cpu().numpy().astype(np.int64), want_key)
    assert np.array_equal(pos[:kept].cpu().numpy().astype(np.int64), want_pos)

    order = np.argsort(want_key, kind="stable")
    sorted_pos = want_pos[order]
    data = (1.0 - rng.random(E)).astype(np.float32)
    divisor = (0.5 + rng.random(N)).astype(np.float32)
    for with_data in (True, False):
        out_row, out_value, out_indptr = capi.coo_block_values(
            key[:kept].contiguous(), pos[:kept].contiguous(), room, to_dev(row, dev),
            to_dev(data, dev) if with_data else None, to_dev(divisor, dev), S)
        assert np.array_equal(out_row.cpu().numpy(), row[sorted_pos])
        w = data[sorted_pos] if with_data else np.ones(sorted_pos.size, np.float32)
        assert np.array_equal(out_value.cpu().numpy(), w / divisor[row[sorted_pos]])
        want_indptr = np.concatenate([[0], np.cumsum(np.bincount(col[sorted_pos], minlength=S))])
        assert np.array_equal(out_indptr.cpu().numpy(), want_indptr)


def test_block_values_without_edges_has_offsets_of_zero(dev):
    empty = torch.empty(0, dtype=torch.int32, device=dev)
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    _, _, indptr = capi.coo_block_values(empty, empty, 64, one, None,
                                         torch.ones(1, dtype=torch.float32, device=dev), 700)
    assert indptr.numel() == 701 and int(indptr.abs().sum()) == 0


def _matrix(dev, n_log, e_log, seed, with_data, tt=torch.int64):
    indptr, indices = rmat_csc_np(1 << n_log, 1 << e_log, seed=seed)
    data = None
    if with_data:
        data = to_dev((1.0 - np.random.default_rng(seed).random(indices.size)).astype(np.float32), dev)
    return gs.Matrix().load_csc(to_dev(indptr, dev), to_dev(indices, dev).to(tt), data)


def _chain(graph, seeds, fanout):
    U = graph._CAPI_Slicing(seeds, 0, _CSC, _COO, False)
    prob = U._CAPI_Sum(1, 2, _CSR)
    picked = torch.ops.gs_ops.list_sampling_with_probs(U._CAPI_GetRows(), prob, fanout, False)[0]
    nodes = torch.cat((seeds, picked)).unique()
    sub = U._CAPI_Slicing(nodes, 1, _CSR, _COO, False)
    sub = sub._CAPI_Divide(prob[nodes], 1, _COO)._CAPI_Normalize(0, _CSC)
    return sub._CAPI_Relabel(), sub._CAPI_GetData("default")


@pytest.mark.parametrize("tt", [torch.int32, torch.int64])
@pytest.mark.parametrize("with_data", [True, False])
@pytest.mark.parametrize("ordered", [True, False])
def test_one_call_layer_equals_the_operator_chain(dev, tt, with_data, ordered):
    """Same frontier, offsets and renamed rows bit for bit; the values bit for bit when the row
    probabilities are (ordered sums), else to 1e-5 -- and the next call draws with the seed the
    chain would have reached."""
    A = _matrix(dev, 13, 18, 3, with_data, tt)
    gs.set_ordered_sums(ordered)
    try:
        for trial, (count, fanout) in enumerate(((300, 256), (1, 64), (2000, 512), (64, 1 << 13))):
            seeds = torch.randperm(1 << 13, device=dev)[:count].to(tt)
            if count == 1:  # a column that has edges
                seeds = A._graph._CAPI_GetCSC()[0].diff().argmax().reshape(1).to(tt)
            gs.set_seed(70 + trial)
            (frontier, num_src, num_dst, indptr, rows, e_ids, fmt), data = _chain(A._graph, seeds, fanout)
            after_chain = torch.ops.gs_ops.list_sampling_with_probs(
                torch.arange(100, device=dev), torch.ones(100, device=dev), 5, False)[0]
            gs.set_seed(70 + trial)
            parts = A._graph._CAPI_LayerwiseBlockIfFused(seeds, fanout)
            after_call = torch.ops.gs_ops.list_sampling_with_probs(
                torch.arange(100, device=dev), torch.ones(100, device=dev), 5, False)[0]
            assert torch.equal(after_chain, after_call)
            if fanout == 1 << 13:  # every row is picked: more nodes than the one-workgroup sort takes
                assert parts == []
                continue
            got_frontier, got_indptr, got_rows, got_values = parts
            assert fmt == "csc" and num_dst == count and num_src == got_frontier.numel()
            assert torch.equal(got_frontier, frontier)
            assert torch.equal(got_indptr, indptr)
            assert torch.equal(got_rows, rows)
            torch.testing.assert_close(got_values, data[e_ids] if e_ids is not None else data,
                                       rtol=0.0 if ordered else 1e-5, atol=0.0)
    finally:
        gs.set_ordered_sums(False)


def test_one_call_layer_against_the_oracle(dev):
    """The layer from the oracle's operators on host arrays, picks made by the device's own
    row probabilities (float sums in another order differ in the last bits)."""
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=4)
    data = (1.0 - np.random.default_rng(4).random(indices.size)).astype(np.float32)
    A = gs.Matrix().load_csc(to_dev(indptr, dev), to_dev(indices, dev), to_dev(data, dev))
    N, k = 1 << 12, 128
    seeds = np.random.default_rng(2).permutation(N)[:200].astype(np.int64)
    d_seeds = to_dev(seeds, dev)
    gs.set_ordered_sums(True)  # the same probabilities in both calls
    try:
        prob = A[:, d_seeds].sum(axis=1, powk=2).cpu().numpy()
        gs.set_seed(11)
        frontier, offsets, rows, values = A._graph._CAPI_LayerwiseBlockIfFused(d_seeds, k)
    finally:
        gs.set_ordered_sums(False)
    sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
    picked, _ = O.list_sample_weighted(np.arange(N, dtype=np.int64), prob, k, seed=11)
    nodes = np.unique(np.concatenate([seeds, picked]))
    r_ip, r_col, r_perm = O.coo2csc(si, coo, N, False)
    s_ip, s_row, s_col, s_sel = O.slice_columns(r_ip, r_col, nodes)
    w_div = (data[sel][r_perm][s_sel] / prob[nodes][s_row]).astype(np.float32)
    c_ip, c_row, c_perm = O.coo2csc(s_col, s_row, seeds.size, False)
    col_of = np.repeat(np.arange(seeds.size), np.diff(c_ip))
    col_sum = np.bincount(col_of, weights=w_div[c_perm].astype(np.float64), minlength=seeds.size)
    want_frontier, (want_rows,) = O.relabel([seeds, nodes[c_row]], [nodes[c_row]])
    assert np.array_equal(frontier.cpu().numpy(), want_frontier)
    assert np.array_equal(offsets.cpu().numpy(), c_ip)
    assert np.array_equal(rows.cpu().numpy(), want_rows)
    want_values = w_div[c_perm] / col_sum[col_of]
    np.testing.assert_allclose(values.cpu().numpy(), want_values, rtol=1e-5)


def test_one_call_layer_declines_graphs_it_does_not_take(dev):
    A = _matrix(dev, 10, 14, 5, True)
    seeds = torch.arange(50, device=dev)
    sliced = A[:, torch.arange(600, device=dev)]  # a graph with a column id list
    gs.set_seed(3)
    assert sliced._graph._CAPI_LayerwiseBlockIfFused(seeds, 16) == []
    assert A._graph._CAPI_LayerwiseBlockIfFused(seeds[:0], 16) == []
    assert A._graph._CAPI_LayerwiseBlockIfFused(seeds.to(torch.int32), 16) == []
    # and the helper of the compiled samplers then runs the chain
    gs.set_ordered_sums(True)  # the same bits in both runs
    try:
        gs.set_seed(3)
        want = _chain(sliced._graph, seeds, 16)
        gs.set_seed(3)
        got = passes.layerwise_block(sliced._graph, seeds, 16)
    finally:
        gs.set_ordered_sums(False)
    for a, b in zip(want[0], got[0]):
        assert torch.equal(a, b) if isinstance(a, torch.Tensor) else a == b
    assert torch.equal(want[1], got[1])
