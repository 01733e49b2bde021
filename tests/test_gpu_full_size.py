"""GPU parity at the benchmark configurations' full sizes.

Where the CPU oracle finishes in seconds the comparison is exact (the whole GraphSAGE minibatch,
the whole walk trace, the layer-wise sampler's layer); where it does not, the checks are the
size-independent properties of the operation (every sampled edge exists, positions are distinct
within a row, relabelling inverts through the frontier, absorbing -1) and, for SDDMM, a torch fp32
gather-and-dot of the same tensors.  Graphs come from the seeded on-device R-MAT generator."""
import numpy as np
import pytest
import torch

import graph_sampling_amd as gs
from graph_sampling_amd import _COO, _CSC, _CSR, capi, rmat
from oracle import oracle as O

pytestmark = pytest.mark.gpu

FANOUTS = (15, 10, 5)


def _host(t):
    return t.cpu().numpy().astype(np.int64)


@pytest.fixture(scope="module")
def sage_graph(dev):
    """R-MAT 2.45 M nodes / 124 M edges, int64 offsets, int32 ids (the GraphSAGE configuration)."""
    indptr, indices = rmat.rmat_csc(2_450_000, 124_000_000, seed=0, device=dev, index_dtype=torch.int32)
    return indptr, indices, _host(indptr), _host(indices)


def test_graphsage_minibatch_full_size_matches_oracle(dev, sage_graph):
    """Two [15,10,5] minibatches of 1024 seeds through the Graph API: every layer's offsets,
    relabelled ids and frontier equal the oracle's on the same seeds and draws."""
    indptr, indices, h_indptr, h_indices = sage_graph
    g = gs.Graph(False)
    g._CAPI_LoadCSC(indptr, indices)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    torch.ops.gs_ops._CAPI_SetSeed(500)
    call = 500
    for _ in range(2):
        seeds = torch.randperm(2_450_000, generator=gen, device=dev)[:1024].to(torch.int32)
        h_seeds = _host(seeds)
        for k in FANOUTS:
            sub = g._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
            frontier, n_src, n_dst, ptr, idx, e_ids, fmt = sub._CAPI_Relabel()
            sp, _, rows, _ = O.sample_uniform(h_indptr, h_indices, h_seeds, k, False, seed=call,
                                              with_coo=False)
            call += 1
            want_frontier, (want_idx,) = O.relabel([h_seeds, rows], [rows])
            assert fmt == "csc" and n_dst == h_seeds.size and n_src == want_frontier.size
            assert np.array_equal(_host(ptr), sp)
            assert np.array_equal(_host(idx), want_idx)
            assert np.array_equal(_host(frontier), want_frontier)
            assert sub._CAPI_GetNumEdges() == rows.size
            assert np.array_equal(_host(sub._CAPI_GetCSC()[1]), rows)
            seeds, h_seeds = frontier, want_frontier


@pytest.mark.parametrize("replace", [False, True])
def test_sampler_properties_full_size(dev, sage_graph, replace):
    """2^18 columns, fanout 10, checked without the oracle: counts, positions inside the column,
    ids read from those positions, distinct positions per row without replacement; and the
    one-launch and two-phase entry points agree bit for bit."""
    indptr, indices, _, _ = sage_graph
    S, k = 1 << 18, 10
    gen = torch.Generator(device=dev)
    gen.manual_seed(9)
    cols = torch.randint(0, 2_450_000, (S,), generator=gen, device=dev).to(torch.int32)
    sub_indptr, sub, sel, coo = capi.sample_uniform_fused(indptr, indices, cols, k, replace, seed=4,
                                                          with_coo=True)
    nnz = int(sub_indptr[-1].item())
    sub, sel, coo = sub[:nnz], sel[:nnz], coo[:nnz].long()
    c = cols.long()
    start, deg = indptr[c], indptr[c + 1] - indptr[c]
    want_cnt = torch.where(deg > 0, torch.full_like(deg, k), deg) if replace else deg.clamp(max=k)
    assert torch.equal(sub_indptr[1:] - sub_indptr[:-1], want_cnt)
    assert torch.equal(coo, torch.repeat_interleave(torch.arange(S, device=dev), want_cnt))
    assert bool(((sel >= start[coo]) & (sel < start[coo] + deg[coo])).all())
    assert torch.equal(indices[sel], sub)
    if not replace:
        assert torch.unique(coo * (1 << 31) + (sel - start[coo])).numel() == nnz
        full = deg <= k  # rows that fit are copied in order
        first = sub_indptr[:-1][full]
        assert torch.equal(sel[first[deg[full] > 0]], start[full][deg[full] > 0])
    two = capi.sample_uniform(indptr, indices, cols, k, replace, seed=4, with_coo=True)
    assert torch.equal(two[0], sub_indptr)
    assert torch.equal(two[1][:nnz], sub) and torch.equal(two[2][:nnz], sel)


def test_relabel_properties_full_size(dev, sage_graph):
    """1.3 M ids with heavy repetition: the frontier is the distinct ids, seeds first, in
    first-occurrence order, and relabelling inverts through it."""
    indptr, indices, _, _ = sage_graph
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    seeds = torch.randperm(2_450_000, generator=gen, device=dev)[:100_000].to(torch.int32)
    sub_indptr, sub, _, _ = capi.sample_uniform_fused(indptr, indices, seeds, 12, False, seed=8)
    sub = sub[:int(sub_indptr[-1].item())]
    frontier, num, (rel,) = capi.unique_relabel([seeds, sub], [sub])
    U = int(num.item())
    frontier = frontier[:U]
    assert torch.equal(frontier[:seeds.numel()], seeds)
    assert U == torch.unique(torch.cat([seeds, sub])).numel() == torch.unique(frontier).numel()
    assert torch.equal(frontier[rel.long()], sub)
    # first-occurrence order: the rank of an id's first appearance grows with its position
    cat = torch.cat([seeds, sub]).long()
    first_pos = torch.full((2_450_000,), cat.numel(), dtype=torch.int64, device=dev)
    first_pos.scatter_reduce_(0, cat, torch.arange(cat.numel(), device=dev), reduce="amin")
    fp = first_pos[frontier.long()]
    assert bool((fp[1:] > fp[:-1]).all())


def test_random_walk_full_size_matches_oracle(dev):
    """R-MAT 4 M nodes / 200 M edges, 1 M uniform starts, 80 steps: the 81 M-entry trace equals the
    oracle's; independently, every step is an edge of the graph and -1 is absorbing."""
    N, E, n, L = 4_000_000, 200_000_000, 1_000_000, 80
    indptr, indices = rmat.rmat_csc(N, E, seed=0, device=dev, index_dtype=torch.int32)
    gen = torch.Generator(device=dev)
    gen.manual_seed(4)
    starts = torch.randint(0, N, (n,), generator=gen, device=dev).to(torch.int32)
    trace = capi.random_walk(indptr, indices, starts, L, seed=21)
    want = O.random_walk(_host(indptr), _host(indices), _host(starts), L, seed=21)
    assert np.array_equal(_host(trace), want)
    t = trace.view(L + 1, n).long()
    assert torch.equal(t[0], starts.long())
    dead = t == -1
    assert bool((dead[1:] | ~dead[:-1]).all())  # once -1, always -1
    # a live walker only dies in a column without neighbours
    deg = indptr[1:] - indptr[:-1]
    died = dead[1:] & ~dead[:-1]
    assert bool((deg[t[:-1][died]] == 0).all())
    # edge existence, step by step, against the sorted list of (column, neighbour) keys
    col_of_edge = torch.repeat_interleave(torch.arange(N, device=dev), deg)
    keys = torch.sort(col_of_edge * N + indices.long()).values
    del col_of_edge
    for s in range(0, L, 8):
        c, r = t[s:s + 8].reshape(-1), t[s + 1:s + 9].reshape(-1)
        live = r >= 0
        q = c[live] * N + r[live]
        pos = torch.searchsorted(keys, q).clamp(max=keys.numel() - 1)
        assert torch.equal(keys[pos], q)


def test_metapath_walk_full_size_matches_oracle(dev):
    """Four bipartite relations (R-MAT 1 M x 2 M, 50 M edges each), metapath of 4 repeated 4 times,
    1 M walkers, through HeteroGraph: the trace equals the oracle's."""
    U, I_, T = 1_000_000, 2_000_000, 1_000_000
    rel = {  # name: (src type size = rows, dst type size = columns)
        "item_to_user": (I_, U), "user_to_item": (U, I_), "tag_to_item": (T, I_), "item_to_tag": (I_, T)}
    graphs, host = {}, {}
    for i, (name, (n_src, n_dst)) in enumerate(rel.items()):
        ip, ix = rmat.rmat_csc(n_dst, 50_000_000, seed=10 + i, device=dev, num_src_nodes=n_src)
        g = gs.Graph(False)
        g._CAPI_LoadCSC(ip, ix)
        graphs[name], host[name] = g, (_host(ip), _host(ix))
    hg = gs.HeteroGraph()
    # a walker sitting on a column of relation (src, name, dst) moves to one of its rows
    hg._CAPI_LoadFromHomo(["user", "item", "tag"],
                          [("item", "item_to_user", "user"), ("user", "user_to_item", "item"),
                           ("tag", "tag_to_item", "item"), ("item", "item_to_tag", "tag")],
                          [graphs[n] for n in rel])
    # users -> items -> tags -> items -> users, four times
    path = ["item_to_user", "tag_to_item", "item_to_tag", "user_to_item"] * 4
    gen = torch.Generator(device=dev)
    gen.manual_seed(6)
    starts = torch.randint(0, U, (1_000_000,), generator=gen, device=dev)
    torch.ops.gs_ops._CAPI_SetSeed(77)
    trace = hg._CAPI_MetapathRandomWalkFused(starts, path)
    names = list(rel)
    want = O.metapath_walk([host[n][0] for n in names], [host[n][1] for n in names],
                           [names.index(p) for p in path], _host(starts), seed=77)
    assert trace.shape == (1_000_000, 17)
    assert np.array_equal(_host(trace.reshape(-1)), want)


def test_ladies_layer_full_size_matches_oracle(dev, sage_graph):
    """One LADIES layer on the 2.45 M-node graph with fp32 edge weights in (0, 1]: slice 512 seed
    columns, row probability = sum of squared weights, weighted list sampling of 512 of the 2.45 M
    rows, row slice, divide, normalise -- each stage against the oracle."""
    indptr, indices32, h_indptr, h_indices = sage_graph
    N = 2_450_000
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    weights = 1.0 - torch.rand(indices32.numel(), generator=gen, device=dev)
    h_w = weights.cpu().numpy()
    m = gs.Matrix()
    m.load_csc(indptr, indices32.long(), weights)
    seeds = torch.randperm(N, generator=gen, device=dev)[:512]
    h_seeds = _host(seeds)
    Uu = m[:, seeds]
    prob = Uu.sum(axis=1, powk=2)
    sp, coo, si, sel = O.slice_columns(h_indptr, h_indices, h_seeds)
    want_prob = O.coo_sum(si, None, h_w[sel], 2, N)
    np.testing.assert_allclose(prob.cpu().numpy(), want_prob, rtol=1e-5)

    gs.set_seed(31)
    row_ids = Uu.row_ids(remove_isolated=False)
    selected, idx = torch.ops.gs_ops._CAPI_ListSamplingWithProbs(row_ids, prob, 512, False)
    w_sel, w_idx = O.list_sample_weighted(np.arange(N), prob.cpu().numpy(), 512, seed=31)
    assert np.array_equal(_host(idx), w_idx) and np.array_equal(_host(selected), w_sel)
    assert (want_prob[w_idx] > 0).all()

    nodes = torch.cat([seeds, selected]).unique()
    h_nodes = _host(nodes)
    subU = Uu[nodes, :]
    r_ip, r_col, r_perm = O.coo2csc(si, coo, N, False)
    s_ip, s_row, s_col, s_sel = O.slice_columns(r_ip, r_col, h_nodes)
    w_data = h_w[sel][r_perm][s_sel]
    assert subU.get_num_edges() == s_col.size
    assert np.array_equal(subU.get_data().cpu().numpy(), w_data)
    div = subU.divide(prob[nodes], axis=1)
    w_div = w_data / want_prob[h_nodes][s_row]
    np.testing.assert_allclose(div.get_data().cpu().numpy(), w_div, rtol=1e-5)
    norm = div.normalize(axis=0)
    col_sum = np.bincount(s_col, weights=w_div.astype(np.float64), minlength=h_seeds.size)
    np.testing.assert_allclose(norm.get_data().cpu().numpy(), w_div / col_sum[s_col], rtol=1e-4)


def test_sddmm_dot_on_sampled_blocks_full_size(dev, sage_graph):
    """u_dot_v with 64-dim fp32 node features over the sampled edges of a [15,10,5] minibatch
    (global row ids into a 2.45 M x 64 feature matrix), against a torch fp32 gather-and-dot; 1e-5
    relative, the tolerance the dot product's summation order allows."""
    indptr, indices, _, _ = sage_graph
    N = 2_450_000
    gen = torch.Generator(device=dev)
    gen.manual_seed(12)
    feat = torch.randn(N, 64, generator=gen, device=dev)
    m = gs.Matrix()
    m.load_csc(indptr, indices.long())
    seeds = torch.randperm(N, generator=gen, device=dev)[:1024]
    gs.set_seed(3)
    for k in FANOUTS:
        sub = m.fused_columnwise_slicing_sampling(seeds, k, False)
        rows = sub.row_indices()                  # global ids of the sampled neighbours
        g = sub._graph
        ptr = g._CAPI_GetCSC()[0]
        col_local = torch.repeat_interleave(torch.arange(seeds.numel(), device=dev), ptr[1:] - ptr[:-1])
        rhs = feat[seeds]
        out = torch.zeros(rows.numel(), 1, device=dev)
        g._CAPI_SDDMM("dot", feat, rhs, out, 0, 2, _CSC)
        want = (feat[rows] * rhs[col_local]).sum(-1, keepdim=True)
        torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-5)
        seeds = sub.all_indices()


def test_segment_sums_and_column_expansion_full_size(dev, sage_graph):
    """Per-column sum of w^2 and per-column normalisation over all 124 M edges (columns from empty
    to 297 k edges, so every path of the segment kernels runs: by lane, by chunk, pieces across
    chunks), and the CSC -> COO column expansion of the whole graph.  The CPU oracle sums in edge
    order, which at this size is neither fast nor what a 300 k-term fp32 sum should be compared
    with; the checks are a float64 segment reduction of the same data (1e-5 relative), exactness
    of columns of at most 16 edges against an fp32 sequential sum, run-to-run identity, and
    "every non-empty column's normalised weights add up to 1"."""
    indptr, indices, h_indptr, _ = sage_graph
    N, E = indptr.numel() - 1, indices.numel()
    gen = torch.Generator(device=dev)
    gen.manual_seed(21)
    w = 1.0 - torch.rand(E, generator=gen, device=dev)
    lens = indptr[1:] - indptr[:-1]
    out = torch.empty(N, device=dev)
    capi.segment_sum(indptr, None, None, w, 2, out)
    ref = torch.segment_reduce(w.double() ** 2, "sum", lengths=lens, initial=0.0)
    assert bool((out[lens == 0] == 0).all())
    rel = ((out.double() - ref).abs() / ref.clamp(min=1e-300))[lens > 0]
    assert float(rel.max()) < 1e-5
    again = torch.empty(N, device=dev)
    capi.segment_sum(indptr, None, None, w, 2, again)
    assert torch.equal(out, again)
    # short columns: the sequential fp32 sum, bit for bit (a sample of them on the host)
    short = torch.nonzero((lens > 0) & (lens <= 16)).flatten()[:20000].cpu().numpy()
    h_w = w.cpu().numpy()
    h_out = out.cpu().numpy()
    for c in short[::50]:
        acc = np.float32(0)
        for x in h_w[h_indptr[c]:h_indptr[c + 1]]:
            acc = np.float32(acc + np.float32(x * x))
        assert h_out[c] == acc
    norm = torch.empty(E, device=dev)
    capi.segment_normalize(indptr, None, w, norm)
    totals = torch.segment_reduce(norm.double(), "sum", lengths=lens, initial=0.0)
    assert float((totals[lens > 0] - 1.0).abs().max()) < 1e-4
    seg = torch.repeat_interleave(torch.arange(N, device=dev), lens)
    col = capi.csc2coo(indptr, E, torch.int32)
    assert torch.equal(col.long(), seg)
    picks = torch.randint(0, E, (1_000_000,), generator=gen, device=dev)
    want = w[picks].double() / torch.segment_reduce(w.double(), "sum", lengths=lens, initial=0.0)[seg[picks]]
    assert float(((norm[picks].double() - want).abs() / want).max()) < 1e-5


# ------------------------------------------------ configuration 5: 111 M nodes / 1.6 B edges
LARGE_NODES, LARGE_EDGES = 111_000_000, 1_600_000_000


@pytest.fixture(scope="module")
def large_graph(dev):
    """R-MAT 111 M nodes / 1.6 B edges, int64 offsets, int32 ids, 64-d fp32 node features
    (0.89 + 6.4 + 28.4 GB on the device; nothing of it is copied to the host)."""
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 120 * (1 << 30):
        pytest.skip("needs about 120 GB of free device memory (graph, features, generator scratch)")
    indptr, indices = rmat.rmat_csc(LARGE_NODES, LARGE_EDGES, seed=0, device=dev,
                                    index_dtype=torch.int32)
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    features = torch.rand(LARGE_NODES, 64, generator=gen, device=dev) - 0.5
    yield indptr, indices, features
    del indptr, indices, features
    torch.cuda.empty_cache()


def _oracle_layer(indptr, indices, cols_dev, h_cols, k, seed):
    """One layer by the oracle on the columns' own small graph (tests/util.py)."""
    from tests.util import columns_as_a_graph
    h_ptr, h_idx = columns_as_a_graph(indptr, indices, cols_dev)
    sp, _, rows, _ = O.sample_uniform(h_ptr, h_idx, np.arange(h_cols.size, dtype=np.int64), k,
                                      False, seed=seed, with_coo=False)
    frontier, (renamed,) = O.relabel([h_cols, rows], [rows])
    return sp, rows, frontier, renamed


def test_large_graph_minibatch_relabel_and_u_dot_v(dev, large_graph):
    """Configuration 5 through the calls of the reference's samplers: per layer the fused slice +
    sample of 1024 seeds' frontier, u_dot_v of the 64-d features on the sampled block
    (examples/as-gcn/train_minibatch.py:39-41 computes its attention the same way: source
    features by global row id, destination features by column), then Relabel.  Ids are bit-exact
    against the oracle, the dot products within 1e-5 of a torch gather-and-dot."""
    indptr, indices, features = large_graph
    g = gs.Graph(False)
    g._CAPI_LoadCSC(indptr, indices)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    seeds = torch.randperm(LARGE_NODES, generator=gen, device=dev)[:1024].to(torch.int32)
    h_seeds = _host(seeds)
    torch.ops.gs_ops._CAPI_SetSeed(900)
    total = 0
    for l, k in enumerate(FANOUTS):
        sub = g._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
        sp, rows, want_frontier, want_idx = _oracle_layer(indptr, indices, seeds, h_seeds, k, 900 + l)
        E = sub._CAPI_GetNumEdges()
        assert E == rows.size
        out = torch.zeros(E, 1, device=dev)
        rhs = features[seeds.long()]
        sub._CAPI_SDDMM("dot", features, rhs, out, 0, 2, _CSC)
        got_ptr, got_rows = sub._CAPI_GetCSC()[:2]
        assert np.array_equal(_host(got_ptr), sp) and np.array_equal(_host(got_rows), rows)
        col = torch.repeat_interleave(torch.arange(seeds.numel(), device=dev),
                                      got_ptr[1:] - got_ptr[:-1])
        want = (features[got_rows.long()] * rhs[col]).sum(-1, keepdim=True)
        assert torch.allclose(out, want, rtol=1e-5, atol=1e-6)
        frontier, n_src, n_dst, ptr, idx, e_ids, fmt = sub._CAPI_Relabel()
        assert fmt == "csc" and n_dst == h_seeds.size and n_src == want_frontier.size
        assert np.array_equal(_host(ptr), sp)
        assert np.array_equal(_host(idx), want_idx)
        assert np.array_equal(_host(frontier), want_frontier)
        total += E
        seeds, h_seeds = frontier, want_frontier
    assert total > 100_000  # a real minibatch: about 150 k sampled edges on this graph


def test_large_graph_whole_minibatch_call_and_block_sddmm(dev, large_graph):
    """The same configuration through one _CAPI_SampleLayers call (every layer queued on the
    device), then u_dot_v on each relabelled block with the features gathered by the frontier."""
    indptr, indices, features = large_graph
    g = gs.Graph(False)
    g._CAPI_LoadCSC(indptr, indices)
    gen = torch.Generator(device=dev)
    gen.manual_seed(12)
    for rep in range(2):
        seeds = torch.randperm(LARGE_NODES, generator=gen, device=dev)[:1024].to(torch.int32)
        torch.ops.gs_ops._CAPI_SetSeed(40 + 3 * rep)
        parts = g._CAPI_SampleLayers(seeds, list(FANOUTS), False)
        cols, h_cols = seeds, _host(seeds)
        for l, k in enumerate(FANOUTS):
            frontier, offsets, renamed = parts[3 * l:3 * l + 3]
            sp, rows, want_frontier, want_idx = _oracle_layer(indptr, indices, cols, h_cols, k,
                                                              40 + 3 * rep + l)
            assert np.array_equal(_host(offsets), sp)
            assert np.array_equal(_host(renamed), want_idx)
            assert np.array_equal(_host(frontier), want_frontier)
            h = features[frontier.long()]
            out = torch.zeros(renamed.numel(), 1, device=dev)
            capi.sddmm_csc("dot", offsets, renamed, None, None, h, h[:offsets.numel() - 1], out,
                           0, 2, 64, 64, 1, 64)
            col = torch.repeat_interleave(torch.arange(offsets.numel() - 1, device=dev),
                                          offsets[1:] - offsets[:-1])
            want = (features[torch.from_numpy(rows).to(dev)] * features[cols.long()][col]).sum(-1, keepdim=True)
            assert torch.allclose(out, want, rtol=1e-5, atol=1e-6)
            cols, h_cols = frontier, want_frontier


def _check_weighted_minibatch(dev, indptr, indices, weights, num_nodes, first_seed):
    """One [15, 10, 5] x 1024 minibatch on a graph that carries fp32 edge weights, through
    _CAPI_SampleLayers and through the per-layer calls: ids against the oracle bit for bit, and
    every layer's data equal to weights[select_index] (reference src/graph.cc:544-557), the
    oracle's select_index taken to positions of the whole graph."""
    from tests.util import columns_as_a_graph
    g = gs.Graph(False)
    g._CAPI_LoadCSC(indptr, indices)
    g._CAPI_SetData(weights)
    gen = torch.Generator(device=dev)
    gen.manual_seed(first_seed)
    seeds = torch.randperm(num_nodes, generator=gen, device=dev)[:1024].to(indices.dtype)
    torch.ops.gs_ops._CAPI_SetSeed(first_seed)
    parts = g._CAPI_SampleLayers(seeds, list(FANOUTS), False)
    assert len(parts) == 4 * len(FANOUTS)
    torch.ops.gs_ops._CAPI_SetSeed(first_seed)
    cols, h_cols, total = seeds, _host(seeds), 0
    for l, k in enumerate(FANOUTS):
        h_ptr, h_idx, pos = columns_as_a_graph(indptr, indices, cols, with_positions=True)
        sp, _, rows, sel = O.sample_uniform(h_ptr, h_idx, np.arange(h_cols.size, dtype=np.int64),
                                            k, False, seed=first_seed + l, with_coo=False)
        want_frontier, (want_idx,) = O.relabel([h_cols, rows], [rows])
        want_data = weights[pos[torch.from_numpy(sel).to(dev)]]
        sub = g._CAPI_FusedColumnwiseSlicingSampling(cols, k, False)
        r = sub._CAPI_Relabel()
        for frontier, offsets, renamed, data in (parts[4 * l:4 * l + 4],
                                                 (r[0], r[3], r[4], sub._CAPI_GetData("default"))):
            assert np.array_equal(_host(offsets), sp)
            assert np.array_equal(_host(renamed), want_idx)
            assert np.array_equal(_host(frontier), want_frontier)
            assert torch.equal(data, want_data)
        total += rows.size
        cols, h_cols = parts[4 * l], want_frontier
    return total


def test_large_graph_with_edge_weights_keeps_the_queued_path(dev, large_graph):
    """Configuration 5 in full: the 111 M / 1.6 B graph WITH its fp32 edge
    weights attached (6.4 GB)."""
    indptr, indices, _ = large_graph
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    weights = 1.0 - torch.rand(indices.numel(), generator=gen, device=dev)
    assert _check_weighted_minibatch(dev, indptr, indices, weights, LARGE_NODES, 500) > 100_000
    del weights


def test_config_2_graph_with_edge_weights(dev, sage_graph):
    """The same on configuration 2's graph (2.45 M nodes / 124 M edges, int32 ids) with weights,
    which is configuration 3's graph."""
    indptr, indices = sage_graph[:2]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    weights = 1.0 - torch.rand(indices.numel(), generator=gen, device=dev)
    assert _check_weighted_minibatch(dev, indptr, indices, weights, 2_450_000, 600) > 200_000


def test_large_graph_sampler_properties(dev, large_graph):
    """2^18 columns of the 1.6 B-edge graph (positions up to 1.6 * 10^9 in `indices`): counts,
    positions inside the column, ids read from those positions, distinct positions per row."""
    indptr, indices, _ = large_graph
    S, k = 1 << 18, 10
    gen = torch.Generator(device=dev)
    gen.manual_seed(9)
    cols = torch.randint(0, LARGE_NODES, (S,), generator=gen, device=dev).to(torch.int32)
    sub_indptr, sub, sel, coo = capi.sample_uniform_fused(indptr, indices, cols, k, False, seed=4,
                                                          with_coo=True)
    nnz = int(sub_indptr[-1].item())
    sub, sel, coo = sub[:nnz], sel[:nnz], coo[:nnz].long()
    c = cols.long()
    start, deg = indptr[c], indptr[c + 1] - indptr[c]
    assert torch.equal(sub_indptr[1:] - sub_indptr[:-1], deg.clamp(max=k))
    assert bool(((sel >= start[coo]) & (sel < start[coo] + deg[coo])).all())
    assert int(sel.max()) > (1 << 30)
    assert torch.equal(indices[sel], sub)
    assert torch.unique(coo * (1 << 31) + (sel - start[coo])).numel() == nnz


# ------------------------------------------------ configuration 1 at its exact shape
def test_config_1_exact_shape_matches_oracle(dev):
    """R-MAT 2^17 nodes / 2^21 edges, int64 offsets, int32 ids, two layers [10, 5], 512 seeds,
    relabel per block: through the per-layer calls and through the one-call minibatch."""
    n = 1 << 17
    indptr, indices = rmat.rmat_csc(n, 1 << 21, seed=0, device=dev, index_dtype=torch.int32)
    h_indptr, h_indices = _host(indptr), _host(indices)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(indptr, indices)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    for rep in range(3):
        seeds = torch.randperm(n, generator=gen, device=dev)[:512].to(torch.int32)
        first = 70 + 2 * rep
        torch.ops.gs_ops._CAPI_SetSeed(first)
        parts = g._CAPI_SampleLayers(seeds, [10, 5], False)
        torch.ops.gs_ops._CAPI_SetSeed(first)
        cols, h_cols = seeds, _host(seeds)
        for l, k in enumerate((10, 5)):
            sub = g._CAPI_FusedColumnwiseSlicingSampling(cols, k, False)
            frontier, n_src, n_dst, ptr, idx, e_ids, fmt = sub._CAPI_Relabel()
            sp, _, rows, _ = O.sample_uniform(h_indptr, h_indices, h_cols, k, False, seed=first + l,
                                              with_coo=False)
            want_frontier, (want_idx,) = O.relabel([h_cols, rows], [rows])
            for got in ((frontier, ptr, idx), parts[3 * l:3 * l + 3]):
                assert np.array_equal(_host(got[0]), want_frontier)
                assert np.array_equal(_host(got[1]), sp)
                assert np.array_equal(_host(got[2]), want_idx)
            cols, h_cols = frontier, want_frontier
