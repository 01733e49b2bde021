"""GPU parity: the super-batch helpers (encode / decode / offsets, concat / split, per-batch
unique and COO relabel, batched COO filters, index search) vs the numpy oracle, through the
C ABI and through torch.ops.gs_ops / Graph."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu

ID_DTYPES = [torch.int64, torch.int32]


def _np(t):
    return t.cpu().numpy().astype(np.int64)


def _ptr(sizes):
    return np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("sizes", [[5], [0, 3, 0, 0, 7], [300, 1, 0, 5000, 257, 256]])
def test_encode_decode_offsets(dev, sizes, idt):
    ptr = _ptr(sizes)
    enc = 1 << 20
    data = np.random.default_rng(len(sizes)).integers(0, enc, size=ptr[-1]).astype(np.int64)
    got = capi.batch_encode(to_dev(data, dev, idt), to_dev(ptr, dev), enc)
    want = O.batch_encode(data, ptr, enc)
    assert np.array_equal(_np(got), want)
    dec, batch = capi.batch_decode(got, enc)
    assert np.array_equal(_np(dec), data)
    assert np.array_equal(_np(batch), np.repeat(np.arange(len(sizes)), sizes))
    g_ptr, g_dec = capi.batch_offsets(got, len(sizes), enc)
    w_ptr, w_dec = O.batch_offsets(want, len(sizes), enc)
    assert np.array_equal(_np(g_ptr), w_ptr) and np.array_equal(w_ptr, ptr)
    assert np.array_equal(_np(g_dec), w_dec)


def test_encode_refuses_what_does_not_fit_32_bits(dev):
    data = torch.zeros(4, dtype=torch.int32, device=dev)
    ptr = torch.tensor([0, 2, 4], device=dev)
    with pytest.raises(capi.GsError, match="32-bit"):
        capi.batch_encode(data, ptr, 1 << 31)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("B,nseg", [(1, 1), (4, 2), (33, 3), (7, 8)])
def test_concat_split_round_trip(dev, B, nseg, idt):
    rng = np.random.default_rng(B * 10 + nseg)
    ptrs = [_ptr(rng.integers(0, 400, size=B)) for _ in range(nseg)]
    datas = [rng.integers(0, 1 << 30, size=p[-1]).astype(np.int64) for p in ptrs]
    d_ptrs = [to_dev(p, dev) for p in ptrs]
    got = capi.batch_concat([to_dev(d, dev, idt) for d in datas], d_ptrs)
    want = O.batch_concat(datas, ptrs)
    for g, w in zip(got, want):
        assert np.array_equal(_np(g), w)
    # and back: with the batch of every item given, and found from the offsets
    for key in (got[1], None):
        back = capi.batch_split(got[0], got[2], key, d_ptrs)
        for b, d in zip(back, datas):
            assert np.array_equal(_np(b), d)
    for b, d in zip(O.batch_split(want[0], want[2], ptrs), datas):
        assert np.array_equal(b, d)


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_ops_concat_split_unique(dev, idt):
    import graph_sampling_amd as gs
    gs.load_library()
    ops = torch.ops.gs_ops
    rng = np.random.default_rng(0)
    ptrs = [_ptr(rng.integers(0, 300, size=9)) for _ in range(2)]
    datas = [rng.integers(0, 200, size=p[-1]).astype(np.int64) for p in ptrs]
    t_d = [to_dev(d, dev, idt) for d in datas]
    t_p = [to_dev(p, dev) for p in ptrs]
    total, key, total_ptr = ops.BatchConcat(t_d, t_p)
    w_total, w_key, w_ptr = O.batch_concat(datas, ptrs)
    assert np.array_equal(_np(total), w_total) and np.array_equal(_np(key), w_key)
    assert np.array_equal(_np(total_ptr), w_ptr)
    outs = [torch.empty_like(d) for d in t_d]
    ops.BatchSplit(total, total_ptr, key, outs, t_p)
    for o, d in zip(outs, datas):
        assert np.array_equal(_np(o), d)
    for name, sort in (("BatchUnique", False), ("BatchUnique2", True)):
        u, u_ptr, u_key = getattr(ops, name)(total, total_ptr)
        w_u, w_uptr, w_ukey = O.batch_unique(w_total, w_ptr, sort=sort)
        assert np.array_equal(_np(u), w_u) and np.array_equal(_np(u_ptr), w_uptr)
        assert np.array_equal(_np(u_key), w_ukey)
    u, u_ptr, u_key = ops.BatchUniqueByKey(total, total_ptr, key)
    assert np.array_equal(_np(u), O.batch_unique(w_total, w_ptr)[0])


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("B", [1, 5, 64, 700])
def test_batch_coo_relabel(dev, B, idt):
    rng = np.random.default_rng(B)
    seeds_ptr = _ptr(rng.integers(0, 50, size=B))
    coo_ptr = _ptr(rng.integers(0, 900 if B < 100 else 60, size=B))
    seeds = rng.integers(0, 500, size=seeds_ptr[-1]).astype(np.int64)
    row = rng.integers(0, 500, size=coo_ptr[-1]).astype(np.int64)
    # columns are mostly seeds of the same batch; some are strangers and come back as -1
    col = rng.integers(0, 500, size=coo_ptr[-1]).astype(np.int64)
    got = capi.batch_coo_relabel(to_dev(seeds, dev, idt), to_dev(seeds_ptr, dev),
                                 to_dev(row, dev, idt), to_dev(col, dev, idt), to_dev(coo_ptr, dev))
    w_u, w_uptr, w_row, w_col = O.batch_coo_relabel(seeds, seeds_ptr, col, row, coo_ptr)
    n_u = int(got[4].item())
    assert n_u == w_u.size
    assert np.array_equal(_np(got[0][:n_u]), w_u) and np.array_equal(_np(got[1]), w_uptr)
    assert np.array_equal(_np(got[2]), w_row) and np.array_equal(_np(got[3]), w_col)
    assert (w_col == -1).any() and (w_row >= 0).all()
    # through the op, with the reference's argument and result order
    import graph_sampling_amd as gs
    gs.load_library()
    u, u_ptr, o_row, o_col, o_ptr = torch.ops.gs_ops.BatchCOORelabel(
        to_dev(seeds, dev, idt), to_dev(seeds_ptr, dev), to_dev(col, dev, idt),
        to_dev(row, dev, idt), to_dev(coo_ptr, dev))
    assert np.array_equal(_np(u), w_u) and np.array_equal(_np(o_row), w_row)
    assert np.array_equal(_np(o_col), w_col) and np.array_equal(_np(o_ptr), coo_ptr)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("B", [0, 1, 6, 40])
def test_coo_filter(dev, B, idt):
    rng = np.random.default_rng(B + 100)
    n = 1 << 10
    if B == 0:
        E, key_ptr, ids_ptr = 20000, None, None
        ids = rng.permutation(n)[:300].astype(np.int64)
    else:
        key_ptr = _ptr(rng.integers(0, 3000, size=B))
        id_sizes = rng.integers(0, 200, size=B)
        ids_ptr = _ptr(id_sizes)
        E = key_ptr[-1]
        ids = np.concatenate([rng.permutation(n)[:s] for s in id_sizes] + [np.empty(0, np.int64)]).astype(np.int64)
    row = rng.integers(0, n, size=E).astype(np.int64)
    col = rng.integers(0, n, size=E).astype(np.int64)
    got = capi.coo_filter(to_dev(row, dev, idt), to_dev(row, dev, idt), to_dev(col, dev, idt),
                          to_dev(ids, dev, idt),
                          None if B == 0 else to_dev(key_ptr, dev),
                          None if B == 0 else to_dev(ids_ptr, dev))
    want = O.coo_filter(row, row, col, ids, key_ptr, ids_ptr)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(_np(g), w)


@pytest.mark.parametrize("B,ids_per_batch", [(0, 50000), (64, 300), (64, 4000), (3000, 40)])
def test_coo_filter_many_edges(dev, B, ids_per_batch):
    """From 2^20 edges on: workgroups that stay, the filter (or its folded copy) in LDS, and the
    batch of an edge found by stepping on from the batch of its tile's first edge."""
    rng = np.random.default_rng(B + ids_per_batch)
    n = 1 << 17
    E = (1 << 20) + 12345
    if B == 0:
        key_ptr = ids_ptr = None
        ids = rng.permutation(n)[:ids_per_batch].astype(np.int64)
    else:
        cuts = np.sort(rng.integers(0, E, size=B - 1))
        key_ptr = np.concatenate([[0], cuts, [E]]).astype(np.int64)
        id_sizes = rng.integers(0, 2 * ids_per_batch, size=B)
        ids_ptr = _ptr(id_sizes)
        ids = np.concatenate([rng.integers(0, n, size=s) for s in id_sizes]).astype(np.int64)
    row = rng.integers(0, n, size=E).astype(np.int64)
    col = rng.integers(0, n, size=E).astype(np.int64)
    got = capi.coo_filter(to_dev(row, dev, torch.int32), to_dev(row, dev, torch.int32),
                          to_dev(col, dev, torch.int32), to_dev(ids, dev, torch.int32),
                          None if B == 0 else to_dev(key_ptr, dev),
                          None if B == 0 else to_dev(ids_ptr, dev))
    want = O.coo_filter(row, row, col, ids, key_ptr, ids_ptr)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(_np(g), w)
    if B == 0:   # closed form
        keep = np.isin(row, ids)
        assert np.array_equal(want[0], row[keep]) and np.array_equal(want[1], col[keep])


@pytest.mark.parametrize("n_data", [3000, 200000])
def test_index_search_many_keys(dev, n_data):
    rng = np.random.default_rng(n_data)
    data = rng.permutation(1 << 20)[:n_data].astype(np.int64)
    keys = rng.integers(0, 1 << 20, size=(1 << 20) + 999).astype(np.int64)
    got = capi.index_search(to_dev(data, dev, torch.int32), to_dev(keys, dev, torch.int32))
    want = O.index_search(data, keys)
    assert np.array_equal(_np(got), want)
    lut = np.full(1 << 20, -1)
    lut[data] = np.arange(n_data)
    assert np.array_equal(want, lut[keys])


def test_ops_coo_slicing_and_global_id(dev):
    import graph_sampling_amd as gs
    gs.load_library()
    ops = torch.ops.gs_ops
    rng = np.random.default_rng(7)
    n, B = 512, 5
    key_ptr = _ptr(rng.integers(100, 2000, size=B))
    id_sizes = rng.integers(1, 100, size=B)
    ids_ptr = _ptr(id_sizes)
    ids = np.concatenate([rng.permutation(n)[:s] for s in id_sizes]).astype(np.int64)
    row = rng.integers(0, n, size=key_ptr[-1]).astype(np.int64)
    col = rng.integers(0, n, size=key_ptr[-1]).astype(np.int64)
    for axis, key in ((0, col), (1, row)):
        r, c, p = ops.BatchCOOSlicing(axis, to_dev(row, dev), to_dev(col, dev), to_dev(key_ptr, dev),
                                      to_dev(ids, dev), to_dev(ids_ptr, dev))
        w = O.coo_filter(key, row, col, ids, key_ptr, ids_ptr)
        assert np.array_equal(_np(r), w[0]) and np.array_equal(_np(c), w[1]) and np.array_equal(_np(p), w[2])
    r, c = ops.COORowSlicingGlobalId(to_dev(row, dev), to_dev(col, dev), to_dev(ids[:50], dev))
    w = O.coo_filter(row, row, col, ids[:50])
    assert np.array_equal(_np(r), w[0]) and np.array_equal(_np(c), w[1])


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_index_search(dev, idt):
    rng = np.random.default_rng(3)
    data = rng.permutation(1 << 16)[:5000].astype(np.int64)
    data[10] = data[3]      # a repeated value reports its last position
    keys = rng.integers(0, 1 << 16, size=20000).astype(np.int64)
    got = capi.index_search(to_dev(data, dev, idt), to_dev(keys, dev, idt))
    want = O.index_search(data, keys)
    assert np.array_equal(_np(got), want)
    assert (want >= 0).any() and (want == -1).any()
    hit = want >= 0
    assert np.array_equal(data[want[hit]], keys[hit])
    import graph_sampling_amd as gs
    gs.load_library()
    assert np.array_equal(_np(torch.ops.gs_ops.index_search(to_dev(data, dev, idt), to_dev(keys, dev, idt))), want)


def test_batch_list_sampling_with_probs(dev):
    import graph_sampling_amd as gs
    gs.load_library()
    rng = np.random.default_rng(5)
    rng_ptr = _ptr([3000, 10, 0, 800])
    probs = (1.0 - rng.random(rng_ptr[-1])).astype(np.float32)
    probs[5:40] = 0.0           # never picked while positive weights remain
    k = 100
    idx, out_ptr = torch.ops.gs_ops.batch_list_sampling_with_probs(
        to_dev(probs, dev), k, False, to_dev(rng_ptr, dev))
    idx, out_ptr = _np(idx), _np(out_ptr)
    assert np.array_equal(out_ptr, [0, 100, 110, 110, 210])
    for b in range(4):
        got = idx[out_ptr[b]:out_ptr[b + 1]]
        assert np.unique(got).size == got.size
        assert ((got >= rng_ptr[b]) & (got < rng_ptr[b + 1])).all()
    assert np.array_equal(idx[100:110], np.arange(3000, 3010))   # a short range is taken whole
    assert not np.isin(idx[:100], np.arange(5, 40)).any()


def test_graph_batch_slicing_split_decode(dev):
    import graph_sampling_amd as gs
    n = 1 << 10
    indptr, indices = rmat_csc_np(n, 1 << 14, seed=11)
    data = np.random.default_rng(0).random(indices.size).astype(np.float32)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    g._CAPI_SetData(to_dev(data, dev))
    nid_ptr = np.array([0, 100, 100, 260], dtype=np.int64)
    n_ids = np.random.default_rng(1).integers(0, n, size=260).astype(np.int64)
    for encoding in (False, True):
        sub, offsets = g._CAPI_BatchSlicing(to_dev(n_ids, dev), to_dev(nid_ptr, dev), 0, gs._CSC,
                                            gs._CSC + gs._COO, False, encoding)
        s_ptr, s_col, s_idx, s_sel = O.slice_columns(indptr, indices, n_ids, True)
        ptr, idx, _ = sub._CAPI_GetCSC()
        assert np.array_equal(_np(ptr), s_ptr)
        assert np.array_equal(_np(offsets), s_ptr[nid_ptr])
        want_idx = O.batch_encode(s_idx, s_ptr[nid_ptr], n) if encoding else s_idx
        assert np.array_equal(_np(idx), want_idx)
        row, col = sub._CAPI_GetBatchCOO()
        assert np.array_equal(_np(row), want_idx) and np.array_equal(_np(col), s_col)
        assert np.array_equal(sub._CAPI_GetData("default").cpu().numpy(), data[s_sel])
        assert np.array_equal(_np(sub._CAPI_GetCols()), O.batch_encode(n_ids, nid_ptr, n))
        assert sub._CAPI_GetNumRows() == 3 * n and sub._CAPI_GetNumCols() == 260
    # Split: pieces of 300 columns, the last one shorter; edge data follows
    pieces = g._CAPI_Split(300)
    assert [p._CAPI_GetNumCols() for p in pieces] == [300, 300, 300, 124]
    for i, p in enumerate(pieces):
        lo, hi = i * 300, min((i + 1) * 300, n)
        ptr, idx, _ = p._CAPI_GetCSC()
        assert np.array_equal(_np(ptr), indptr[lo:hi + 1] - indptr[lo])
        assert np.array_equal(_np(idx), indices[indptr[lo]:indptr[hi]])
        assert np.array_equal(p._CAPI_GetData("default").cpu().numpy(), data[indptr[lo]:indptr[hi]])
    # Decode: ids back to one batch's range
    sub, _ = g._CAPI_BatchSlicing(to_dev(n_ids, dev), to_dev(nid_ptr, dev), 0, gs._CSC, gs._CSC,
                                  True, True)
    rows_before = _np(sub._CAPI_GetRows())
    sub._CAPI_Decode(n)
    assert np.array_equal(_np(sub._CAPI_GetCols()), n_ids)
    assert np.array_equal(_np(sub._CAPI_GetRows()), rows_before % n)


def test_fastgcn_super_batch_equals_batch_by_batch(dev):
    """The flow of the reference's examples/fastgcn/batching.py:70-106 on B small batches at
    once against the same steps done one batch at a time."""
    import graph_sampling_amd as gs
    gs.load_library()
    ops = torch.ops.gs_ops
    n, B, bs = 1 << 11, 6, 64
    indptr, indices = rmat_csc_np(n, 1 << 15, seed=12)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    rng = np.random.default_rng(2)
    seeds = rng.permutation(n)[:B * bs].astype(np.int64)
    seeds_ptr = np.arange(B + 1, dtype=np.int64) * bs
    t_seeds, t_seeds_ptr = to_dev(seeds, dev), to_dev(seeds_ptr, dev)

    sub = g._CAPI_Slicing(t_seeds, 0, gs._CSC, gs._CSC + gs._COO, False)
    _, idx, idx_ptr = sub.GetBatchCSC(t_seeds_ptr)
    encoded = ops.BatchEncode(idx, idx_ptr, n)
    neighbors = torch.unique(encoded)
    nb_ptr, nb_ids = ops.GetBatchOffsets(neighbors, B, n)
    # "selected": every third neighbour of each batch, in encoded form
    keep = torch.arange(neighbors.numel(), device=dev) % 3 == 0
    selected = neighbors[keep]
    coo_row, coo_col = sub.GetBatchCOO()
    s_row, s_col = ops.COORowSlicingGlobalId(encoded, coo_col, selected)
    s_ptr, s_row = ops.GetBatchOffsets(s_row, B, n)
    u, u_ptr, r_row, r_col, r_ptr = ops.BatchCOORelabel(t_seeds, t_seeds_ptr, s_col, s_row, s_ptr)
    # columns of the sliced COO are local to the super-batch (0..B*bs): relabel them as ids of seeds
    u, u_ptr, r_row, r_col = _np(u), _np(u_ptr), _np(r_row), _np(r_col)
    s_ptr = _np(s_ptr)
    nb_ptr, nb_ids, neighbors_np = _np(nb_ptr), _np(nb_ids), _np(neighbors)
    for b in range(B):
        sb = seeds[b * bs:(b + 1) * bs]
        _, cc, ii, _ = O.slice_columns(indptr, indices, sb, True)
        nb = np.unique(ii)
        assert np.array_equal(nb_ids[nb_ptr[b]:nb_ptr[b + 1]], nb)
        sel_b = _np(selected)[(_np(selected) // n) == b] % n
        keep_e = np.isin(ii, sel_b)
        rows_b, cols_b = ii[keep_e], cc[keep_e] + b * bs
        lo, hi = s_ptr[b], s_ptr[b + 1]
        assert np.array_equal(_np(s_row)[lo:hi], rows_b) and np.array_equal(_np(s_col)[lo:hi], cols_b)
        frontier, (w_row, w_col) = O.relabel([sb, rows_b], [rows_b, cols_b])
        assert np.array_equal(u[u_ptr[b]:u_ptr[b + 1]], frontier)
        assert np.array_equal(r_row[lo:hi], w_row) and np.array_equal(r_col[lo:hi], w_col)


def test_batch_relabel_64_bit_ids_narrow_and_fallback(dev):
    """The host layer first tries one-word slots for 64-bit ids and falls back to the two-array
    slots when an id does not fit 32 bits; both give the oracle's result."""
    import graph_sampling_amd as gs
    gs.load_library()
    rng = np.random.default_rng(3)
    B = 5
    seeds_ptr = np.arange(B + 1, dtype=np.int64) * 40
    ids_ptr = np.concatenate([[0], np.cumsum(rng.integers(50, 300, B))]).astype(np.int64)
    for offset in (0, 3_000_000_000, 1 << 34):
        seeds = rng.integers(0, 500, seeds_ptr[-1]).astype(np.int64) + offset
        ids = rng.integers(0, 500, ids_ptr[-1]).astype(np.int64) + offset
        uni, uni_ptr, rel, _ = torch.ops.gs_ops.BatchCSRRelabel(
            to_dev(seeds, dev), to_dev(seeds_ptr, dev), to_dev(ids, dev), to_dev(ids_ptr, dev))
        for b in range(B):
            f, (r,) = O.relabel([seeds[seeds_ptr[b]:seeds_ptr[b + 1]], ids[ids_ptr[b]:ids_ptr[b + 1]]],
                                [ids[ids_ptr[b]:ids_ptr[b + 1]]])
            lo, hi = int(uni_ptr[b]), int(uni_ptr[b + 1])
            assert np.array_equal(uni[lo:hi].cpu().numpy(), f)
            assert np.array_equal(rel[ids_ptr[b]:ids_ptr[b + 1]].cpu().numpy(), r)


def _oracle_super_batch(indptr, indices, seed_sets, fanouts, replace, first_seed, data=None):
    """The super-batch flow by the oracle: one sampler call per layer over the concatenated seeds
    (row r of the call draws as row r), one relabel per minibatch, next seeds = the frontiers."""
    sizes = [s.size for s in seed_sets]
    seeds = np.concatenate(seed_sets).astype(np.int64) if seed_sets else np.empty(0, np.int64)
    sp = _ptr(sizes)
    out = [[] for _ in seed_sets]
    for l, k in enumerate(fanouts):
        sub_ptr, _, rows, sel = O.sample_uniform(indptr, indices, seeds, k, replace,
                                                 seed=first_seed + l, with_coo=False)
        ip = sub_ptr[sp]
        uni, uni_ptr, rel = O.batch_csr_relabel(seeds, sp, rows, ip)
        for b in range(len(seed_sets)):
            out[b] += [uni[uni_ptr[b]:uni_ptr[b + 1]], sub_ptr[sp[b]:sp[b + 1] + 1] - sub_ptr[sp[b]],
                       rel[ip[b]:ip[b + 1]]]
            if data is not None:
                out[b].append(data[sel][ip[b]:ip[b + 1]])
        seeds, sp = uni, uni_ptr
    return out


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("with_data", [False, True])
@pytest.mark.parametrize("sizes,fanouts,replace", [([300, 0, 1, 1024, 77], (4, 3), False),
                                                   ([1024] * 64, (15, 10), False),
                                                   ([50, 60], (3, 3, 3), True)])
def test_sample_layers_batched_equals_the_oracle_flow(dev, idt, with_data, sizes, fanouts, replace):
    """_CAPI_SampleLayersBatched (the super-batch flow inside the C++ layer: fused sampling over
    the concatenated seeds, the batches' edge cuts, one relabel per minibatch in one pass -- through
    the bins from 2^19 items on --, the per-minibatch views) against the oracle doing the same."""
    import graph_sampling_amd as gs
    n = 1 << 15
    indptr, indices = rmat_csc_np(n, 1 << 20, seed=41)
    rng = np.random.default_rng(len(sizes))
    data = (1.0 - rng.random(indices.size)).astype(np.float32) if with_data else None
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, idt))
    if with_data:
        g._CAPI_SetData(to_dev(data, dev))
    seed_sets = [rng.permutation(n)[:s].astype(np.int64) for s in sizes]
    ops = torch.ops.gs_ops
    # first with every layer's relabel queued behind its sampler (sized by the sampler's capacity,
    # one host wait a layer), then with the wait for the edge count too (exact sizes): the same
    # minibatches either way, and from 2^19 items on the first way is the one taken
    for first, no_wait in ((700, True), (710, False)):
        through, repeated = ops._CAPI_BatchedNoWaitCounts()
        ops._CAPI_SetBatchedNoWait(no_wait)
        try:
            gs.set_seed(first)
            got = g._CAPI_SampleLayersBatched([to_dev(s, dev, idt) for s in seed_sets],
                                              list(fanouts), replace)
        finally:
            ops._CAPI_SetBatchedNoWait(True)
        now = ops._CAPI_BatchedNoWaitCounts()
        assert now[0] + now[1] == through + repeated + len(fanouts)  # one count per layer
        if not no_wait:
            assert now[0] == through
        elif idt == torch.int32 and len(sizes) == 64:
            assert now == [through + len(fanouts), repeated]  # 2^19 items and more: all queued
        want = _oracle_super_batch(indptr, indices, seed_sets, fanouts, replace, first, data)
        assert len(got) == len(want)
        for b, (g_b, w_b) in enumerate(zip(got, want)):
            assert len(g_b) == len(w_b)
            for j, (x, y) in enumerate(zip(g_b, w_b)):
                if y.dtype == np.float32:
                    assert np.array_equal(x.cpu().numpy(), y), (b, j)
                else:
                    assert np.array_equal(_np(x), y), (b, j)
    # the Python helper hands back blocks, innermost layer first
    gs.set_seed(700)
    res = gs.sample_blocks_batched(g, [to_dev(s, dev, idt) for s in seed_sets], fanouts, replace)
    want = _oracle_super_batch(indptr, indices, seed_sets, fanouts, replace, 700, data)
    nodes, blocks = res[0]
    assert np.array_equal(_np(nodes), want[0][-(4 if with_data else 3)])
    assert blocks[-1].num_dst_nodes() == sizes[0]


def test_sample_layers_batched_on_a_graph_with_id_maps_goes_minibatch_by_minibatch(dev):
    import graph_sampling_amd as gs
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=13)
    col_ids = np.random.default_rng(1).permutation(1 << 12).astype(np.int64)
    g = gs.Graph(False)
    g._CAPI_LoadCSCWithColIds(to_dev(col_ids, dev), to_dev(indptr, dev), to_dev(indices, dev))
    sets = [to_dev(np.arange(100, dtype=np.int64), dev), to_dev(np.arange(50, 90, dtype=np.int64), dev)]
    gs.set_seed(5)
    got = g._CAPI_SampleLayersBatched(sets, [4], False)
    gs.set_seed(5)
    want = [g._CAPI_SampleLayers(s, [4], False) for s in sets]
    for a, b in zip(got, want):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.parametrize("with_data", [False, True])
def test_super_batches_queued_ahead_equal_the_calls_one_by_one(dev, with_data):
    """_CAPI_QueueSampleLayersBatched: three super-batches, each queued before the one before it
    is collected (and the last two collected out of order), give what three
    _CAPI_SampleLayersBatched calls give under the same seeds; a handle collects once; a graph
    with id maps (minibatch by minibatch inside) goes through the same two halves."""
    import graph_sampling_amd as gs
    n = 1 << 15
    indptr, indices = rmat_csc_np(n, 1 << 20, seed=43)
    rng = np.random.default_rng(9)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev, torch.int32))
    if with_data:
        g._CAPI_SetData(to_dev((1.0 - rng.random(indices.size)).astype(np.float32), dev))
    fanouts = [15, 10]
    groups = [[to_dev(rng.permutation(n)[:s].astype(np.int64), dev, torch.int32) for s in sizes]
              for sizes in ([1024] * 64, [300, 0, 1, 1024, 77], [1024] * 48)]
    gs.set_seed(900)
    want = [g._CAPI_SampleLayersBatched(sets, fanouts, False) for sets in groups]
    gs.set_seed(900)
    h0 = g._CAPI_QueueSampleLayersBatched(groups[0], fanouts, False)
    h1 = g._CAPI_QueueSampleLayersBatched(groups[1], fanouts, False)
    got = [h0.collect()]
    h2 = g._CAPI_QueueSampleLayersBatched(groups[2], fanouts, False)
    last = h2.collect()
    got += [h1.collect(), last]
    for a, b in zip(got, want):
        assert len(a) == len(b)
        for x, y in zip(a, b):
            assert len(x) == len(y) == (4 if with_data else 3) * len(fanouts)
            for u, v in zip(x, y):
                assert torch.equal(u, v)
    with pytest.raises(RuntimeError, match="collected already"):
        h1.collect()
    gs.set_seed(900)
    res = gs.queue_sample_blocks_batched(g, groups[0], fanouts).collect()
    assert len(res) == 64 and torch.equal(res[3][0], want[0][3][-(4 if with_data else 3)])
    # a graph the one launch sequence does not take
    col_ids = to_dev(np.random.default_rng(1).permutation(n).astype(np.int64), dev)
    m = gs.Graph(False)
    m._CAPI_LoadCSCWithColIds(col_ids, to_dev(indptr, dev), to_dev(indices, dev))
    sets = [to_dev(np.arange(100, dtype=np.int64), dev), to_dev(np.arange(50, 90, dtype=np.int64), dev)]
    gs.set_seed(5)
    loop = [m._CAPI_SampleLayers(x, [4], False) for x in sets]
    gs.set_seed(5)
    queued = m._CAPI_QueueSampleLayersBatched(sets, [4], False).collect()
    for a, b in zip(queued, loop):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.parametrize("sizes", [[5], [0, 3, 0, 0, 7], [300, 1, 0, 5000, 257, 256], [0, 0, 0]])
def test_indptr_split_with_cuts_through_the_c_abi(dev, sizes):
    """gs_indptr_split_cuts: the re-based offsets of every batch back to back, and where each
    batch's edges start (indptr[offsets]) from the same launch; closed form in numpy."""
    rng = np.random.default_rng(sum(sizes) + len(sizes))
    cols = int(sum(sizes))
    deg = rng.integers(0, 9, size=cols)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    ptr = _ptr(sizes)
    want = np.concatenate([indptr[ptr[b]:ptr[b + 1] + 1] - indptr[ptr[b]] for b in range(len(sizes))])
    plain = capi.indptr_split(to_dev(indptr, dev), to_dev(ptr, dev))
    out, cuts = capi.indptr_split(to_dev(indptr, dev), to_dev(ptr, dev), with_cuts=True)
    assert np.array_equal(_np(plain), want)
    assert np.array_equal(_np(out), want)
    assert np.array_equal(_np(cuts), indptr[ptr])


def test_offsets_reach_pinned_memory_by_one_launch(dev):
    """gs_post_values / gs_post_value_sets: device arrays arrive in pinned host memory, in order,
    with the mailbox telling how many values were stored."""
    rng = np.random.default_rng(5)
    box = capi.Mailbox()
    for n, k in [(65, 9), (1, 1), (1000, 32), (0, 3)]:
        sets = [rng.integers(-2**62, 2**62, size=n).astype(np.int64) for _ in range(k)]
        got = capi.post_value_sets([to_dev(s, dev) for s in sets], box)
        assert (got.is_pinned() or n == 0) and tuple(got.shape) == (k, n)
        assert np.array_equal(got.numpy(), np.stack(sets) if n else np.zeros((k, 0), np.int64))
        one = capi.post_values(to_dev(sets[0], dev), box)
        assert np.array_equal(one.numpy(), sets[0])
    with pytest.raises(capi.GsError):
        capi.post_value_sets([to_dev(np.zeros(4, np.int64), dev)] * 33, box)


def test_super_batch_reports_a_sampler_that_gave_up(dev):
    """A layer's relabel is queued behind its sampler before anyone has read the sampler's total.
    With the sampler's error word raised from the host (every kernel runs to its end) the total it
    leaves is negative: the relabel's passes leave at once, the call raises, the host layer clears
    the sampler's state behind it, and the next call is right again."""
    import graph_sampling_amd as gs
    n = 1 << 15
    indptr, indices = rmat_csc_np(n, 1 << 20, seed=47)
    rng = np.random.default_rng(4)
    t_ptr = to_dev(indptr, dev)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(t_ptr, to_dev(indices, dev, torch.int32))
    sets = [to_dev(rng.permutation(n)[:1024].astype(np.int64), dev, torch.int32) for _ in range(64)]
    fanouts = [15, 10]
    gs.set_seed(40)
    want = g._CAPI_SampleLayersBatched(sets, fanouts, False)
    torch.ops.gs_ops._CAPI_DebugRaiseLookbackError(t_ptr)
    through, _ = torch.ops.gs_ops._CAPI_BatchedNoWaitCounts()
    with pytest.raises(RuntimeError, match="gave up"):
        g._CAPI_SampleLayersBatched(sets, fanouts, False)
    for _ in range(2):
        gs.set_seed(40)
        got = g._CAPI_SampleLayersBatched(sets, fanouts, False)
        for a, b in zip(got, want):
            for x, y in zip(a, b):
                assert torch.equal(x, y)
    # (the calls that went through did so with every layer's relabel queued behind its sampler)
    assert torch.ops.gs_ops._CAPI_BatchedNoWaitCounts()[0] >= through + 2 * len(fanouts)
