"""GPU parity: random walks and metapath walks through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import rmat_csc_np, to_dev, u32_draws

pytestmark = pytest.mark.gpu


def _tables(indptrs, indicess, dev, idt):
    d_ip = [to_dev(a, dev) for a in indptrs]
    d_ix = [to_dev(a, dev, idt) for a in indicess]
    ip_tab = torch.tensor([t.data_ptr() for t in d_ip], dtype=torch.int64, device=dev)
    ix_tab = torch.tensor([t.data_ptr() for t in d_ix], dtype=torch.int64, device=dev)
    nn_tab = torch.tensor([t.numel() - 1 for t in d_ip], dtype=torch.int64, device=dev)
    return d_ip, d_ix, ip_tab, ix_tab, nn_tab


def test_metapath_reference_unique_path(dev):
    # reference tests/test_hetero_random_walk.cc:29-71: every hop has exactly one choice
    indptr1, indices1 = np.array([0, 0, 1, 2, 3]), np.array([0, 1, 2])   # "follow"
    indptr2, indices2 = np.array([0, 1, 2, 3]), np.array([0, 1, 2])      # "view"
    keep = _tables([indptr1, indptr2], [indices1, indices2], dev, torch.int64)
    metapath = np.array([1, 0, 0], dtype=np.int64)  # view, follow, follow
    seeds = np.array([2, 1], dtype=np.int64)
    trace = capi.metapath_walk(keep[2], keep[3], keep[4], torch.int64, to_dev(metapath, dev), to_dev(seeds, dev),
                               seed=3)
    expected = np.array([2, 1, 2, 1, 1, 0, 0, -1], dtype=np.int64)  # step-major [4][2]
    assert np.array_equal(trace.cpu().numpy(), expected)
    assert np.array_equal(O.metapath_walk([indptr1, indptr2], [indices1, indices2], metapath, seeds,
                                          seed=3), expected)


def test_metapath_reference_multi_path_edges_exist(dev):
    # reference tests/test_hetero_random_walk.cc:74-120
    indptr1, indices1 = np.array([0, 0, 1, 2, 3]), np.array([0, 1, 2])
    indptr2, indices2 = np.array([0, 1, 3, 5]), np.array([0, 0, 1, 2, 3])
    graphs = {0: (indptr1, indices1), 1: (indptr2, indices2)}
    keep = _tables([indptr1, indptr2], [indices1, indices2], dev, torch.int64)
    metapath = np.array([1, 0, 0], dtype=np.int64)
    seeds = np.array([2, 2, 1, 1, 0], dtype=np.int64)
    trace = capi.metapath_walk(keep[2], keep[3], keep[4], torch.int64, to_dev(metapath, dev), to_dev(seeds, dev),
                               seed=11).cpu().numpy().reshape(4, 5)
    for w in range(5):
        for t in range(3):
            src, dst = trace[t, w], trace[t + 1, w]
            if dst == -1:
                continue
            ip, ix = graphs[int(metapath[t])]
            assert dst in ix[ip[src]:ip[src + 1]]
        dead = np.where(trace[:, w] == -1)[0]
        if dead.size:
            assert (trace[dead[0]:, w] == -1).all()  # -1 is absorbing
    want = O.metapath_walk([indptr1, indptr2], [indices1, indices2], metapath, seeds, seed=11)
    assert np.array_equal(trace.reshape(-1), want)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("length", [0, 1, 7, 80])
def test_random_walk_matches_oracle(dev, idt, length):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 15, seed=9)  # avg degree 8, plenty of dead ends
    seeds = np.random.default_rng(length).integers(0, 1 << 12, size=5000).astype(np.int64)
    got = capi.random_walk(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(seeds, dev, idt),
                           length, seed=21)
    want = O.random_walk(indptr, indices, seeds, length, seed=21)
    assert np.array_equal(got.cpu().numpy().astype(np.int64), want)
    if length:
        assert (want == -1).any()
    # layout: flat [L+1][n]; row 0 is the seeds
    assert np.array_equal(want[:seeds.size], seeds)


def test_random_walk_replay(dev):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=10)
    n, L = 3000, 12
    seeds = np.random.default_rng(0).integers(0, 1 << 12, size=n).astype(np.int64)
    replay = u32_draws(n * L, 5)
    got = capi.random_walk(to_dev(indptr, dev), to_dev(indices, dev), to_dev(seeds, dev), L,
                           replay=to_dev(replay, dev))
    want = O.random_walk(indptr, indices, seeds, L, replay=replay)
    assert np.array_equal(got.cpu().numpy(), want)
    # closed form for one live step: indices[indptr[c] + r % deg]
    c = seeds
    deg = indptr[c + 1] - indptr[c]
    step1 = np.where(deg > 0, indices[np.minimum(indptr[c] + replay[:n] % np.maximum(deg, 1), indices.size - 1)], -1)
    assert np.array_equal(want[n:2 * n], step1)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_metapath_walk_rmat(dev, idt):
    rels = [rmat_csc_np(1 << 11, 1 << 14, seed=s) for s in (1, 2, 3)]
    indptrs, indicess = [r[0] for r in rels], [r[1] for r in rels]
    keep = _tables(indptrs, indicess, dev, idt)
    metapath = np.array([0, 1, 2, 1] * 4, dtype=np.int64)
    seeds = np.random.default_rng(3).integers(0, 1 << 11, size=4096).astype(np.int64)
    got = capi.metapath_walk(keep[2], keep[3], keep[4], idt, to_dev(metapath, dev), to_dev(seeds, dev, idt), seed=8)
    want = O.metapath_walk(indptrs, indicess, metapath, seeds, seed=8)
    assert np.array_equal(got.cpu().numpy().astype(np.int64), want)


def test_walk_next_hop_chi_square(dev):
    """Next hop of a degree-d node is uniform over its d neighbours."""
    d, n = 16, 64000
    indptr = np.array([0, d] + [d] * d, dtype=np.int64)  # node 0 has d neighbours 1..d, others none
    indices = np.arange(1, d + 1, dtype=np.int64)
    seeds = np.zeros(n, dtype=np.int64)
    got = capi.random_walk(to_dev(indptr, dev), to_dev(indices, dev), to_dev(seeds, dev), 1, seed=77)
    hop = got.cpu().numpy()[n:]
    counts = np.bincount(hop, minlength=d + 1)[1:].astype(np.float64)
    chi2 = ((counts - n / d) ** 2 / (n / d)).sum()
    assert chi2 < (d - 1) + 5 * np.sqrt(2 * (d - 1)), chi2


def test_walk_out_of_range_seeds_die(dev):
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=13)
    seeds = np.array([5, -1, 1 << 10, 7, (1 << 10) + 999, -7], dtype=np.int64)
    got = capi.random_walk(to_dev(indptr, dev), to_dev(indices, dev), to_dev(seeds, dev), 4, seed=1)
    want = O.random_walk(indptr, indices, seeds, 4, seed=1)
    assert np.array_equal(got.cpu().numpy(), want)
    tr = want.reshape(5, 6)
    assert (tr[1:, [1, 2, 4, 5]] == -1).all()
