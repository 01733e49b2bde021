"""The one entry point that allocates nothing (gs_sample_uniform_fused_static) against the
entry point it is a variant of (gs_sample_uniform_fused), through the C ABI."""
import numpy as np
import pytest
import torch

from graph_sampling_amd import capi
from tests.util import rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu


def _both(indptr, indices, cols, fanout, replace, seed, dev, with_extras):
    S = cols.numel()
    cap = S * fanout
    want = capi.sample_uniform_fused(indptr, indices, cols, fanout, replace, seed=seed,
                                     with_coo=with_extras)
    # outputs start from a pattern, so that a slot the call does not write shows
    out = (torch.full((S + 1,), -7, dtype=torch.int64, device=dev),
           torch.full((cap,), -7, dtype=indices.dtype, device=dev),
           torch.full((cap,), -7, dtype=torch.int64, device=dev) if with_extras else None,
           torch.full((cap,), -7, dtype=indices.dtype, device=dev) if with_extras else None)
    capi.sample_uniform_fused_static(indptr, indices, cols, fanout, replace, out, seed=seed)
    torch.cuda.synchronize()
    n = int(want[0][-1])
    assert n == int(out[0][-1])
    assert torch.equal(want[0], out[0])
    assert torch.equal(want[1][:n], out[1][:n])
    if with_extras:
        assert torch.equal(want[2][:n], out[2][:n])
        assert torch.equal(want[3][:n], out[3][:n])
    return n


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_static_state_sampler_equals_the_sampler_with_a_state_buffer(dev, idt):
    h_indptr, h_indices = rmat_csc_np(1 << 14, 1 << 18, seed=3)
    indptr, indices = to_dev(h_indptr, dev), to_dev(h_indices, dev, idt)
    rng = np.random.default_rng(4)
    # two calls in a row on the same device array, the second with a smaller input: tiles of
    # the first call that the second does not use must not be mistaken for its own
    big = to_dev(rng.integers(0, 1 << 14, size=40_000), dev, idt)
    small = to_dev(rng.integers(0, 1 << 14, size=700), dev, idt)
    n_big = _both(indptr, indices, big, 10, False, 11, dev, True)
    n_small = _both(indptr, indices, small, 10, False, 12, dev, True)
    assert n_big > n_small > 0
    # with replacement, without the optional outputs, one column, no column at all
    _both(indptr, indices, big[:5000], 7, True, 13, dev, False)
    _both(indptr, indices, small[:1], 5, False, 14, dev, False)
    _both(indptr, indices, small[:0], 5, False, 15, dev, False)
    # a third size after a smaller one
    _both(indptr, indices, big[:20_000], 15, False, 16, dev, True)


def test_static_state_sampler_refuses_more_columns_than_its_state_holds(dev):
    h_indptr, h_indices = rmat_csc_np(1 << 10, 1 << 12, seed=1)
    indptr, indices = to_dev(h_indptr, dev), to_dev(h_indices, dev, torch.int32)
    S = (1 << 22) + 1
    cols = torch.zeros(S, dtype=torch.int32, device=dev)
    out = (torch.empty(S + 1, dtype=torch.int64, device=dev),
           torch.empty(S, dtype=torch.int32, device=dev), None, None)
    with pytest.raises(capi.GsError, match="exceed"):
        capi.sample_uniform_fused_static(indptr, indices, cols, 1, False, out, seed=1)
    # and the limit itself is served
    cols = torch.zeros(1 << 22, dtype=torch.int32, device=dev)
    want = capi.sample_uniform_fused(indptr, indices, cols, 1, False, seed=2)
    capi.sample_uniform_fused_static(indptr, indices, cols, 1, False, out, seed=2)
    torch.cuda.synchronize()
    n = int(want[0][-1])
    assert torch.equal(want[0], out[0][:(1 << 22) + 1]) and torch.equal(want[1][:n], out[1][:n])


def test_static_state_sampler_allocates_nothing(dev):
    """Free device memory is the same before and after static calls of several sizes (the
    outputs are made beforehand; the call itself must not reach the allocator)."""
    h_indptr, h_indices = rmat_csc_np(1 << 13, 1 << 17, seed=5)
    indptr, indices = to_dev(h_indptr, dev), to_dev(h_indices, dev, torch.int32)
    sizes = (30_000, 500, 12_000)
    cols = [to_dev(np.random.default_rng(s).integers(0, 1 << 13, size=s), dev, torch.int32)
            for s in sizes]
    outs = [(torch.empty(s + 1, dtype=torch.int64, device=dev),
             torch.empty(s * 8, dtype=torch.int32, device=dev),
             torch.empty(s * 8, dtype=torch.int64, device=dev), None) for s in sizes]
    capi.sample_uniform_fused_static(indptr, indices, cols[0], 8, False, outs[0], seed=1)  # warm-up
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    reserved_before = torch.cuda.memory_reserved(dev)
    for rep in range(3):
        for c, o in zip(cols, outs):
            capi.sample_uniform_fused_static(indptr, indices, c, 8, rep == 1, o, seed=rep)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.cuda.memory_reserved(dev) == reserved_before


def test_static_state_sampler_recovers_after_a_reset(dev):
    """The error word a give-up leaves is in the library's own array: every later call reports
    -1 until gs_sample_uniform_fused_static_reset, after which results are right again."""
    h_indptr, h_indices = rmat_csc_np(1 << 12, 1 << 16, seed=6)
    indptr, indices = to_dev(h_indptr, dev), to_dev(h_indices, dev, torch.int32)
    cols = to_dev(np.random.default_rng(2).integers(0, 1 << 12, size=3000), dev, torch.int32)
    _both(indptr, indices, cols, 6, False, 30, dev, False)
    capi.static_debug_raise(dev)
    out = (torch.empty(3001, dtype=torch.int64, device=dev),
           torch.empty(18000, dtype=torch.int32, device=dev), None, None)
    for seed in (31, 32):  # sticky: both report the failure
        capi.sample_uniform_fused_static(indptr, indices, cols, 6, False, out, seed=seed)
        torch.cuda.synchronize()
        assert int(out[0][-1]) == -1
    capi.static_reset()
    _both(indptr, indices, cols, 6, False, 33, dev, False)
    _both(indptr, indices, cols[:100], 6, False, 34, dev, True)


def test_static_state_sampler_recorded_into_a_graph_is_right_on_every_replay(dev):
    """One static call recorded into a HIP graph, the column ids rewritten in place between the
    replays, eager static calls of other sizes in between (they leave other epochs in the shared
    state): every replay equals gs_sample_uniform_fused on the same columns."""
    h_indptr, h_indices = rmat_csc_np(1 << 13, 1 << 17, seed=7)
    indptr, indices = to_dev(h_indptr, dev), to_dev(h_indices, dev, torch.int32)
    rng = np.random.default_rng(8)
    S, k = 20_000, 10
    cols = to_dev(rng.integers(0, 1 << 13, size=S), dev, torch.int32)
    out = (torch.full((S + 1,), -7, dtype=torch.int64, device=dev),
           torch.full((S * k,), -7, dtype=torch.int32, device=dev),
           torch.full((S * k,), -7, dtype=torch.int64, device=dev), None)
    other = to_dev(rng.integers(0, 1 << 13, size=900), dev, torch.int32)
    other_out = (torch.empty(901, dtype=torch.int64, device=dev),
                 torch.empty(900 * k, dtype=torch.int32, device=dev), None, None)
    capi.static_init()
    capi.sample_uniform_fused_static(indptr, indices, other, k, False, other_out, seed=1)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.sample_uniform_fused_static(indptr, indices, cols, k, False, out, seed=21)
    for rep in range(3):
        cols.copy_(to_dev(rng.integers(0, 1 << 13, size=S), dev, torch.int32))
        for o in out[:3]:
            o.fill_(-7)
        capi.sample_uniform_fused_static(indptr, indices, other, k, False, other_out, seed=rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = capi.sample_uniform_fused(indptr, indices, cols, k, False, seed=21)
        n = int(want[0][-1])
        assert int(out[0][-1]) == n > 0
        assert torch.equal(want[0], out[0])
        assert torch.equal(want[1][:n], out[1][:n]) and torch.equal(want[2][:n], out[2][:n])
    # an eager call after the recorded one still works (the epoch count was left at "fill first")
    _both(indptr, indices, cols[:5000], k, False, 40, dev, True)
