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


def test_rewrites_fuse_slice_with_sample_and_share_one_relabel():
    c = jit.compile(graphsage, (gs.Matrix(), torch.arange(4), [10, 5]))
    t = _targets(c)
    assert t.count(passes.FUSED) == 2
    assert "_CAPI_Slicing" not in t and "_CAPI_Sampling" not in t
    assert t.count("_CAPI_Relabel") == 2 and "_CAPI_AllValidNode" not in t
    # the fused call takes (seeds, fanout, replace) of the pair it replaces
    fused = [n for n in c.gm.graph.nodes if n.target == passes.FUSED]
    assert [n.args[2:] for n in fused] == [(10, False), (5, False)]


def test_slice_with_a_second_consumer_is_not_fused():
    def sampler(A, seeds):
        sliced = A[:, seeds]
        return sliced.columnwise_sampling(3, False).all_indices(), sliced.row_ids()

    t = _targets(jit.compile(sampler, (gs.Matrix(), torch.arange(4))))
    assert "_CAPI_Slicing" in t and "_CAPI_Sampling" in t and passes.FUSED not in t


def test_weighted_and_row_slices_are_left_alone():
    c = jit.compile(ladies, (gs.Matrix(), torch.arange(4), [64, 64]))
    t = _targets(c)
    assert t.count("_CAPI_Slicing") == 4 and t.count("_CAPI_Relabel") == 2
    assert "_CAPI_AllValidNode" not in t and t.count("_CAPI_Sum") == 2


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
