"""The sampler compiler: traces and rewrites need no device (graph handles are symbolic)."""
import pytest
import torch

import graph_sampling_amd as gs
from graph_sampling_amd import jit
from graph_sampling_amd.jit import passes


def graphsage(A, seeds, fanouts):
    blocks = []
    for k in fanouts:
        sub = A[:, seeds].columnwise_sampling(k, False)
        seeds = sub.all_indices()
        blocks.insert(0, sub.to_dgl_block())
    return seeds, blocks


def ladies(A, seeds, fanouts):
    # the flow of examples/ladies/ladies_raw.py:8-27
    ret = []
    for fanout in fanouts:
        U = A[:, seeds]
        prob = U.sum(axis=1, powk=2)
        selected, _ = torch.ops.gs_ops.list_sampling_with_probs(U.row_ids(unique=False), prob,
                                                                fanout, False)
        nodes = torch.cat((seeds, selected)).unique()
        subU = U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0)
        seeds = subU.all_indices()
        ret.insert(0, subU.to_dgl_block())
    return seeds, ret


def _targets(compiled):
    return [str(n.target) for n in compiled.gm.graph.nodes if n.op == "call_method"]


def test_raw_trace_records_the_calls_of_the_matrix_api():
    raw = jit.compile(graphsage, (gs.Matrix(), torch.arange(4), [10, 5]), passes=())
    t = _targets(raw)
    assert t.count("_CAPI_Slicing") == 2 and t.count("_CAPI_Sampling") == 2
    assert t.count("_CAPI_Relabel") == 2 and t.count("_CAPI_AllValidNode") == 2


PER_LAYER = tuple(p for p in passes.DEFAULT if p is not passes.chain_sampled_layers)


def test_rewrites_fuse_slice_with_sample_and_share_one_relabel():
    c = jit.compile(graphsage, (gs.Matrix(), torch.arange(4), [10, 5]), passes=PER_LAYER)
    t = _targets(c)
    assert t.count(passes.FUSED) == 2
    assert "_CAPI_Slicing" not in t and "_CAPI_Sampling" not in t
    assert t.count("_CAPI_Relabel") == 2 and "_CAPI_AllValidNode" not in t
    # the fused call takes (seeds, fanout, replace) of the pair it replaces
    fused = [n for n in c.gm.graph.nodes if n.target == passes.FUSED]
    assert [n.args[2:] for n in fused] == [(10, False), (5, False)]


def _functions(compiled):
    return [n for n in compiled.gm.graph.nodes if n.op == "call_function"]


def test_consecutive_layers_become_one_chain_call():
    c = jit.compile(graphsage, (gs.Matrix(), torch.arange(4), [10, 5, 3]))
    assert _targets(c) == []  # no per-layer call is left
    chains = [n for n in _functions(c) if n.target is passes.sample_layer_chain]
    assert len(chains) == 1
    graph, seeds, fanouts, replace = chains[0].args
    assert fanouts == [10, 5, 3] and replace is False
    # the three blocks are made of layers 0, 1, 2 of the chain, and the sampler's seeds are
    # the last layer's frontier
    blocks = [n for n in _functions(c) if n.target is gs.block.make_block]
    assert [b.args[0].args[0].args for b in blocks] == [(chains[0], l) for l in range(3)]
    nodes, made = c.gm.graph.output_node().args[0]
    assert made == blocks[::-1] and nodes.args == (blocks[2].args[0], 0)


def test_layers_are_chained_only_where_the_loop_is_the_plain_one():
    def one_layer(A, seeds):
        return A[:, seeds].columnwise_sampling(3, False).to_dgl_block()

    def sample_kept(A, seeds):  # the sampled matrix itself is asked for its rows as well
        blocks, rows = [], []
        for k in (4, 2):
            sub = A[:, seeds].columnwise_sampling(k, False)
            rows.append(sub.row_ids())
            seeds = sub.all_indices()
            blocks.append(sub.to_dgl_block())
        return blocks, rows

    def two_graphs(A, B, seeds):
        sub = A[:, seeds].columnwise_sampling(4, False)
        nxt = B[:, sub.all_indices()].columnwise_sampling(2, False)
        return sub.to_dgl_block(), nxt.to_dgl_block()

    def mixed_replace(A, seeds):
        sub = A[:, seeds].columnwise_sampling(4, False)
        nxt = A[:, sub.all_indices()].columnwise_sampling(2, True)
        return sub.to_dgl_block(), nxt.to_dgl_block()

    for sampler, args in ((one_layer, (gs.Matrix(), torch.arange(4))),
                          (sample_kept, (gs.Matrix(), torch.arange(4))),
                          (two_graphs, (gs.Matrix(), gs.Matrix(), torch.arange(4))),
                          (mixed_replace, (gs.Matrix(), torch.arange(4)))):
        c = jit.compile(sampler, args)
        assert not [n for n in _functions(c) if n.target is passes.sample_layer_chain], sampler
        assert passes.FUSED in _targets(c)


def test_a_chain_may_start_behind_other_work_and_two_chains_stay_apart():
    def sampler(A, seeds, more):
        first = graphsage(A, torch.cat((seeds, more)), [4, 2])
        second = graphsage(A, more, [3, 3, 3])
        return first, second

    c = jit.compile(sampler, (gs.Matrix(), torch.arange(4), torch.arange(2)))
    chains = [n for n in _functions(c) if n.target is passes.sample_layer_chain]
    assert [n.args[2] for n in chains] == [[4, 2], [3, 3, 3]]
    assert passes.FUSED not in _targets(c)


def test_slice_with_a_second_consumer_is_not_fused():
    def sampler(A, seeds):
        sliced = A[:, seeds]
        return sliced.columnwise_sampling(3, False).all_indices(), sliced.row_ids()

    t = _targets(jit.compile(sampler, (gs.Matrix(), torch.arange(4))))
    assert "_CAPI_Slicing" in t and "_CAPI_Sampling" in t and passes.FUSED not in t


NO_LAYERWISE = tuple(p for p in passes.DEFAULT if p is not passes.fuse_layerwise_block)


def test_weighted_and_row_slices_are_left_alone():
    c = jit.compile(ladies, (gs.Matrix(), torch.arange(4), [64, 64]), passes=NO_LAYERWISE)
    t = _targets(c)
    assert t.count("_CAPI_Slicing") == 4 and t.count("_CAPI_Relabel") == 2
    assert "_CAPI_AllValidNode" not in t and t.count("_CAPI_Sum") == 2


def test_a_layer_of_a_layerwise_sampler_becomes_one_call():
    c = jit.compile(ladies, (gs.Matrix(), torch.arange(4), [64, 32]))
    assert _targets(c) == []  # nothing of the operator chain is left
    layers = [n for n in _functions(c) if n.target is passes.layerwise_block]
    assert [n.args[2] for n in layers] == [64, 32]
    # the second layer's seeds are the first layer's frontier; the blocks are made of the
    # layers' (relabel, data) pairs
    first_relabel = [u for u in layers[0].users if u.args[1] == 0][0]
    assert layers[1].args[1].args == (first_relabel, 0)
    blocks = [n for n in _functions(c) if n.target is gs.block.make_block]
    assert [b.args[0].args for b in blocks] == [(l, 0) for l in layers]
    assert [b.args[1].args for b in blocks] == [(l, 1) for l in layers]


def test_a_layer_whose_parts_are_used_elsewhere_stays_a_chain():
    def keeps_the_probabilities(A, seeds, fanouts):
        U = A[:, seeds]
        prob = U.sum(axis=1, powk=2)
        picked, _ = torch.ops.gs_ops.list_sampling_with_probs(U.row_ids(unique=False), prob,
                                                              fanouts[0], False)
        nodes = torch.cat((seeds, picked)).unique()
        sub = U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0)
        return sub.to_dgl_block(), prob

    def other_power(A, seeds, fanouts):
        U = A[:, seeds]
        prob = U.sum(axis=1, powk=1)
        picked, _ = torch.ops.gs_ops.list_sampling_with_probs(U.row_ids(unique=False), prob,
                                                              fanouts[0], False)
        nodes = torch.cat((seeds, picked)).unique()
        return U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0).to_dgl_block()

    for sampler in (keeps_the_probabilities, other_power):
        c = jit.compile(sampler, (gs.Matrix(), torch.arange(4), [64]))
        assert not [n for n in _functions(c) if n.target is passes.layerwise_block], sampler
        assert _targets(c).count("_CAPI_Slicing") == 2


def test_repeated_queries_are_made_once_but_samples_stay_apart():
    def sampler(A, seeds):
        sub = A[:, seeds]
        a = sub.row_ids()
        b = sub.row_ids()
        s1 = sub.columnwise_sampling(2, False).row_indices()
        s2 = sub.columnwise_sampling(2, False).row_indices()
        return a, b, s1, s2

    t = _targets(jit.compile(sampler, (gs.Matrix(), torch.arange(4))))
    assert t.count("_CAPI_GetValidRows") == 1 and t.count("_CAPI_Sampling") == 2


def test_dead_code_keeps_calls_that_change_their_receiver():
    def sampler(A, seeds, w):
        sub = A[:, seeds]
        sub.row_ids()            # unused query: removed
        sub.set_data(w)          # changes `sub`: kept
        return sub.get_data()

    t = _targets(jit.compile(sampler, (gs.Matrix(), torch.arange(4), torch.ones(3))))
    assert "_CAPI_SetData" in t and "_CAPI_GetValidRows" not in t


def test_frozen_arguments_must_not_change():
    c = jit.compile(graphsage, (gs.Matrix(), torch.arange(4), [10, 5]))
    with pytest.raises(ValueError, match="frozen"):
        c(gs.Matrix(), torch.arange(4), [10, 10])
    with pytest.raises(TypeError):
        c(gs.Matrix(), torch.arange(4))
