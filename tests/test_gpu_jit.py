"""GPU: a compiled sampler returns what the sampler itself returns on the same seeds."""
import numpy as np
import pytest
import torch

import graph_sampling_amd as gs
from graph_sampling_amd import jit
from graph_sampling_amd.jit import passes
from tests.test_jit import graphsage, ladies
from tests.util import rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu


def _matrix(dev, n_log, e_log, seed, with_data=False):
    indptr, indices = rmat_csc_np(1 << n_log, 1 << e_log, seed=seed)
    data = None
    if with_data:
        data = to_dev((1.0 - np.random.default_rng(seed).random(indices.size)).astype(np.float32), dev)
    return gs.Matrix().load_csc(to_dev(indptr, dev), to_dev(indices, dev), data)


def _same_block(a, b, rtol=0.0):
    assert a.num_src_nodes() == b.num_src_nodes() and a.num_dst_nodes() == b.num_dst_nodes()
    assert torch.equal(a.srcdata["_ID"], b.srcdata["_ID"])
    for x, y in zip(a.edges(), b.edges()):  # a fused layer is CSC, an unfused one COO: same edges
        assert torch.equal(x, y)
    assert ("w" in a.edata) == ("w" in b.edata)
    if "w" in a.edata:
        torch.testing.assert_close(a.edata["w"], b.edata["w"], rtol=rtol, atol=0.0)


@pytest.mark.parametrize("with_data", [False, True])
@pytest.mark.parametrize("chained", [False, True])
def test_compiled_graphsage_equals_eager(dev, with_data, chained):
    A = _matrix(dev, 13, 17, 1, with_data)
    rewrites = tuple(p for p in passes.DEFAULT if chained or p is not passes.chain_sampled_layers)
    compiled = jit.compile(graphsage, (A, torch.arange(4, device=dev), [10, 5]), passes=rewrites)
    assert ("sample_layer_chain" if chained else passes.FUSED) in compiled.code
    for trial in range(3):  # replays: fresh seeds and sizes on the same trace
        seeds = torch.randperm(1 << 13, device=dev)[:200 + 50 * trial]
        gs.set_seed(40 + trial)
        want_nodes, want_blocks = graphsage(A, seeds, [10, 5])
        gs.set_seed(40 + trial)
        got_nodes, got_blocks = compiled(A, seeds, [10, 5])
        assert torch.equal(got_nodes, want_nodes)
        for g, w in zip(got_blocks, want_blocks):
            _same_block(g, w)


@pytest.mark.parametrize("replace", [False, True])
def test_chained_layers_of_three_on_a_root_and_on_a_slice(dev, replace):
    """The chain call takes a root graph in one call of the C++ layer and a row slice (a graph
    with an id map, whose columns are still all the nodes) layer by layer: both give the
    per-layer sampler's minibatch, and the next call draws with the seed the loop would have
    reached."""
    def sampler(A, seeds, fanouts):
        blocks = []
        for k in fanouts:
            sub = A[:, seeds].columnwise_sampling(k, replace)
            seeds = sub.all_indices()
            blocks.insert(0, sub.to_dgl_block())
        return seeds, blocks

    root = _matrix(dev, 14, 19, 3)
    fanouts = [15, 10, 5]
    compiled = jit.compile(sampler, (root, torch.arange(4, device=dev), fanouts))
    assert "sample_layer_chain(" in compiled.code and passes.FUSED not in compiled.code
    # on a graph with a row id list the sampler itself orders the next seeds by that list, the
    # rewritten one by the block (merge_relabel_and_all_indices): the yardstick there is the
    # rewritten sampler without the chain
    per_layer = jit.compile(sampler, (root, torch.arange(4, device=dev), fanouts),
                            passes=tuple(p for p in passes.DEFAULT
                                         if p is not passes.chain_sampled_layers))
    # (the fused operator reads a CSC: the rows are sliced on that format and kept in it)
    kept = torch.arange(0, 1 << 14, 2, device=dev)
    sliced = gs.Matrix(root._graph._CAPI_Slicing(kept, 1, gs._CSC, gs._CSC, False))
    for A in (root, sliced):
        for trial, count in enumerate((1024, 1, 3000)):
            seeds = torch.randperm(1 << 13, device=dev)[:count]
            gs.set_seed(90 + trial)
            want = [(sampler if A is root else per_layer)(A, seeds, fanouts) for _ in range(2)]
            gs.set_seed(90 + trial)
            got = [compiled(A, seeds, fanouts) for _ in range(2)]
            for (got_nodes, got_blocks), (want_nodes, want_blocks) in zip(got, want):
                assert torch.equal(got_nodes, want_nodes)
                for g, w in zip(got_blocks, want_blocks):
                    _same_block(g, w)


def ladies_one_frontier(A, seeds, fanouts):
    """`ladies` with the rewrite done by hand: the next layer's seeds are the block's own
    source ids.  After a row slice `all_indices()` lists the kept rows in the order of the
    slice's id list, `Relabel()` in edge order (src/graph.cc:757-778 against :782-839), so the
    merged sampler is the one whose layers agree on the node order."""
    ret = []
    for fanout in fanouts:
        U = A[:, seeds]
        prob = U.sum(axis=1, powk=2)
        selected, _ = torch.ops.gs_ops.list_sampling_with_probs(U.row_ids(unique=False), prob,
                                                                fanout, False)
        nodes = torch.cat((seeds, selected)).unique()
        block = U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0).to_dgl_block()
        seeds = block.srcdata["_ID"]
        ret.insert(0, block)
    return seeds, ret


@pytest.mark.parametrize("ordered", [True, False])
def test_compiled_ladies_equals_eager(dev, ordered):
    """With ordered sums the row probabilities are the same bits in both runs and so is every
    weight; without, they are sums by float atomics, equal to rounding (1e-5 relative, the
    bar for float results)."""
    gs.set_ordered_sums(ordered)
    try:
        _compiled_ladies_equals_eager(dev, 0.0 if ordered else 1e-5)
    finally:
        gs.set_ordered_sums(False)


def _compiled_ladies_equals_eager(dev, rtol):
    A = _matrix(dev, 12, 16, 2, with_data=True)
    seeds = torch.randperm(1 << 12, device=dev)[:128]
    # without the merge the replay is the sampler as written
    plain = jit.compile(ladies, (A, torch.arange(4, device=dev), [64, 64]),
                        passes=(passes.fuse_slicing_and_sampling, passes.common_subexpressions,
                                passes.dead_code))
    merged = jit.compile(ladies, (A, torch.arange(4, device=dev), [64, 64]),
                         passes=tuple(p for p in passes.DEFAULT if p is not passes.fuse_layerwise_block))
    one_call = jit.compile(ladies, (A, torch.arange(4, device=dev), [64, 64]))
    assert "layerwise_block" in one_call.code and "layerwise_block" not in merged.code
    for compiled, eager in ((plain, ladies), (merged, ladies_one_frontier),
                            (one_call, ladies_one_frontier)):
        gs.set_seed(5)
        want_nodes, want_blocks = eager(A, seeds, [64, 64])
        gs.set_seed(5)
        got_nodes, got_blocks = compiled(A, seeds, [64, 64])
        assert torch.equal(got_nodes, want_nodes)
        for g, w in zip(got_blocks, want_blocks):
            _same_block(g, w, rtol)
    # either way the same set of nodes is reached
    gs.set_seed(5)
    a = ladies(A, seeds, [64])[0]
    gs.set_seed(5)
    b = ladies_one_frontier(A, seeds, [64])[0]
    assert torch.equal(a.sort().values, b.sort().values)


def test_compiled_sampler_on_another_graph_and_matrix_results(dev):
    def one_hop(A, seeds):
        return A[:, seeds]  # a Matrix comes back as a Matrix

    A, B = _matrix(dev, 10, 14, 3), _matrix(dev, 10, 14, 4)
    compiled = jit.compile(one_hop, (A, torch.arange(4, device=dev)))
    seeds = torch.arange(100, device=dev)
    for M in (A, B):  # the graph is an argument of the trace, not part of it
        got = compiled(M, seeds)
        assert isinstance(got, gs.Matrix)
        assert torch.equal(got.row_indices(), M[:, seeds].row_indices())


def test_compiled_metapath_walk(dev):
    def walk(H, seeds, metapath):
        return H.metapath_random_walk_fused(seeds, metapath)

    a, b = _matrix(dev, 11, 15, 6), _matrix(dev, 11, 15, 7)
    hm = gs.HeteroMatrix()
    hm.load_from_homo(["a", "b"], [("a", "r0", "b"), ("b", "r1", "a")], [a, b])
    seeds = torch.randint(0, 1 << 11, (300,), device=dev)
    compiled = jit.compile(walk, (hm, seeds, ["r0", "r1", "r0"]))
    gs.set_seed(12)
    want = walk(hm, seeds, ["r0", "r1", "r0"])
    gs.set_seed(12)
    assert torch.equal(compiled(hm, seeds, ["r0", "r1", "r0"]), want)
