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
