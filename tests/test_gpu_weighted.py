"""GPU parity: weighted (A-Res) neighbour sampling and list sampling vs the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import rmat_csc_np, to_dev, u32_draws

pytestmark = pytest.mark.gpu


def _weighted_gpu(dev, indptr, indices, probs, cols, k, idt=torch.int64, seed=0, replay=None, replay_ptr=None):
    dcols = None if cols is None else to_dev(cols, dev, idt)
    sp, si, sel, coo = capi.sample_weighted(to_dev(indptr, dev), to_dev(indices, dev, idt),
                                            to_dev(probs, dev), dcols, k, seed=seed,
                                            replay=None if replay is None else to_dev(replay, dev),
                                            replay_ptr=None if replay_ptr is None else to_dev(replay_ptr, dev),
                                            with_coo=True)
    n = int(sp[-1].item())
    return sp.cpu().numpy(), coo[:n].cpu().numpy().astype(np.int64), si[:n].cpu().numpy().astype(np.int64), sel[:n].cpu().numpy()


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("k", [1, 10, 25, 40, 96])
@pytest.mark.parametrize("fused", [True, False])
def test_weighted_free_running_matches_oracle(dev, idt, k, fused):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=11)  # hubs above the 2048-edge chunk size
    rng = np.random.default_rng(k)
    probs = (1.0 - rng.random(indices.size)).astype(np.float32)
    probs[rng.integers(0, indices.size, 500)] = 0.0  # weight <= 0: never beats a positive weight
    cols = None
    if fused:
        cols = rng.integers(0, indptr.size - 1, size=2000).astype(np.int64)
        cols[:6] = np.argsort(np.diff(indptr))[-6:]
    got = _weighted_gpu(dev, indptr, indices, probs, cols, k, idt, seed=99)
    want = O.sample_weighted(indptr, indices, probs, cols, k, seed=99)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_weighted_replay_matches_oracle(dev):
    indptr, indices = rmat_csc_np(1 << 11, 1 << 16, seed=12)
    k = 12
    probs = (1.0 - np.random.default_rng(1).random(indices.size)).astype(np.float32)
    rp = O.weighted_replay_ptr(indptr, None, k)
    replay = u32_draws(int(rp[-1]), 9)
    got = _weighted_gpu(dev, indptr, indices, probs, None, k, replay=replay, replay_ptr=rp)
    want = O.sample_weighted(indptr, indices, probs, None, k, replay=replay)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_weighted_hub_many_chunks(dev):
    degs = np.array([5, 100000, 0, 3000, 40], dtype=np.int64)
    indptr = np.concatenate([[0], np.cumsum(degs)])
    rng = np.random.default_rng(2)
    indices = rng.integers(0, 1 << 20, int(indptr[-1])).astype(np.int64)
    probs = rng.random(indices.size, dtype=np.float32) + 0.01
    cols = np.array([1, 3, 1, 0, 2, 4], dtype=np.int64)
    got = _weighted_gpu(dev, indptr, indices, probs, cols, 15, seed=5)
    want = O.sample_weighted(indptr, indices, probs, cols, 15, seed=5)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


@pytest.mark.parametrize("k", [1, 9, 63, 64, 65, 96])
def test_weighted_degrees_around_the_selection_paths(dev, k):
    # 256 edges: the last column a wave selects where it finds it; 257 .. 2048: one chunk that
    # the chunk pass finishes by itself; 2049 and up: several chunks and a merge (4196 edges
    # with fanout 96 leave 3 * 96 candidates, 40000 edges with fanout 96 more than the 2048 the
    # register-resident merge holds).  Fanouts on both sides of the 64 lanes (the floor for
    # dropping candidates comes from the lanes' maxima, and exists only up to 64), equal
    # weights everywhere in one column (keys differ by the draws only) and a column whose
    # positive weights are fewer than the fanout.
    degs = np.array([0, 1, k, k + 1, 255, 256, 257, 1000, 2047, 2048, 2049, 4196, 40000, 300, 600],
                    dtype=np.int64)
    indptr = np.concatenate([[0], np.cumsum(degs)])
    rng = np.random.default_rng(k)
    indices = rng.integers(0, 1 << 20, int(indptr[-1])).astype(np.int64)
    probs = (1.0 - rng.random(indices.size)).astype(np.float32)
    probs[indptr[13]:indptr[14]] = 0.25                      # all weights equal
    probs[indptr[14]:indptr[15]] = 0.0                       # ... and few positive ones
    probs[indptr[14] + rng.permutation(600)[:5]] = 0.5
    rp = O.weighted_replay_ptr(indptr, None, k)
    replay = u32_draws(int(rp[-1]), k)
    for idt in (torch.int64, torch.int32):
        got = _weighted_gpu(dev, indptr, indices, probs, None, k, idt, replay=replay, replay_ptr=rp)
        want = O.sample_weighted(indptr, indices, probs, None, k, replay=replay)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)
        got = _weighted_gpu(dev, indptr, indices, probs, None, k, idt, seed=31)
        want = O.sample_weighted(indptr, indices, probs, None, k, seed=31)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)


def test_weighted_special_cases(dev):
    # one dominant weight is always selected; equal weights -> uniform inclusion
    d, k, trials = 30, 5, 3000
    indptr = np.array([0, d], dtype=np.int64)
    indices = np.arange(d, dtype=np.int64)
    cols = np.zeros(trials, dtype=np.int64)
    probs = np.full(d, 1e-3, dtype=np.float32)
    probs[17] = 1e6
    _, _, si, _ = _weighted_gpu(dev, indptr, indices, probs, cols, k, seed=1)
    assert (si.reshape(trials, k) == 17).any(axis=1).all()
    assert (si.reshape(trials, k)[:, 0] == 17).mean() > 0.99  # and it comes first (largest key)
    probs = np.ones(d, dtype=np.float32)
    _, _, si, _ = _weighted_gpu(dev, indptr, indices, probs, cols, k, seed=2)
    counts = np.bincount(si, minlength=d).astype(np.float64)
    expect = trials * k / d
    chi2 = ((counts - expect) ** 2 / (expect * (1 - k / d))).sum()
    assert chi2 < (d - 1) + 5 * np.sqrt(2 * (d - 1)), chi2


def test_weighted_first_pick_proportional_to_weight(dev):
    """A-Res: the largest key belongs to item i with probability w_i / sum(w)."""
    w = np.array([1, 2, 3, 4, 10], dtype=np.float32)
    trials = 20000
    indptr = np.array([0, 5], dtype=np.int64)
    cols = np.zeros(trials, dtype=np.int64)
    _, _, si, _ = _weighted_gpu(dev, indptr, np.arange(5, dtype=np.int64), w, cols, 2, seed=3)
    first = si.reshape(trials, 2)[:, 0]
    counts = np.bincount(first, minlength=5).astype(np.float64)
    expect = trials * w / w.sum()
    chi2 = ((counts - expect) ** 2 / expect).sum()
    assert chi2 < 4 + 5 * np.sqrt(8), chi2


# --------------------------------------------------------------- list sampling
@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_list_uniform_reference_cases(dev, idt):
    # reference tests/test_listsampling.cc:7-40
    data = np.arange(1000, dtype=np.int64)
    d = to_dev(data, dev, idt)
    sel, idx = capi.list_sample_uniform(d, 2000, True, seed=1)
    assert sel.numel() == 2000 and np.unique(sel.cpu().numpy()).size <= 1000
    sel, idx = capi.list_sample_uniform(d, 999, False, seed=1)
    assert np.unique(sel.cpu().numpy()).size == 999
    w_sel, w_idx = O.list_sample_uniform(data, 999, False, seed=1)
    assert np.array_equal(sel.cpu().numpy().astype(np.int64), w_sel) and np.array_equal(idx.cpu().numpy(), w_idx)


@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("n,k", [(10, 3), (5000, 512), (200000, 2000)])
def test_list_uniform_matches_oracle(dev, replace, n, k):
    data = np.random.default_rng(n).integers(0, 1 << 30, n).astype(np.int64)
    sel, idx = capi.list_sample_uniform(to_dev(data, dev), k, replace, seed=7)
    w_sel, w_idx = O.list_sample_uniform(data, k, replace, seed=7)
    assert np.array_equal(sel.cpu().numpy(), w_sel) and np.array_equal(idx.cpu().numpy(), w_idx)
    ndraws = k if replace else n - k
    replay = u32_draws(ndraws, 4)
    sel, idx = capi.list_sample_uniform(to_dev(data, dev), k, replace, replay=to_dev(replay, dev))
    w_sel, w_idx = O.list_sample_uniform(data, k, replace, replay=replay)
    assert np.array_equal(sel.cpu().numpy(), w_sel) and np.array_equal(idx.cpu().numpy(), w_idx)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,k", [(10, 3), (5000, 512), (300000, 2000), (300000, 8192), (2500000, 512)])
def test_list_weighted_matches_oracle(dev, idt, n, k):
    rng = np.random.default_rng(n + k)
    data = rng.integers(0, 1 << 30, n).astype(np.int64)
    probs = rng.random(n, dtype=np.float32)
    probs[rng.integers(0, n, max(1, n // 10))] = 0.0   # never selected while positive weights remain
    sel, idx = capi.list_sample_weighted(to_dev(data, dev, idt), to_dev(probs, dev), k, seed=13)
    w_sel, w_idx = O.list_sample_weighted(data, probs, k, seed=13)
    assert np.array_equal(idx.cpu().numpy(), w_idx)
    assert np.array_equal(sel.cpu().numpy().astype(np.int64), w_sel)
    assert (probs[w_idx] > 0).all()


def test_list_weighted_massive_ties(dev):
    # all weights zero: every key is -inf, ties resolve to the lowest positions
    n, k = 50000, 100
    data = np.arange(n, dtype=np.int64) * 3
    probs = np.zeros(n, dtype=np.float32)
    sel, idx = capi.list_sample_weighted(to_dev(data, dev), to_dev(probs, dev), k, seed=1)
    assert np.array_equal(idx.cpu().numpy(), np.arange(k))
    assert np.array_equal(O.list_sample_weighted(data, probs, k, seed=1)[1], np.arange(k))


@pytest.mark.parametrize("n,k,positive", [
    (300000, 512, 100),     # fewer positive weights than picks: the rest by position
    (300000, 512, 511),
    (2500000, 2000, 700),
    (3000, 2999, 10),
    (70000, 8192, 8000),    # more picked items above the k-th key's class than one sort holds
])
def test_list_weighted_with_few_positive_weights(dev, n, k, positive):
    rng = np.random.default_rng(n + positive)
    data = rng.integers(0, 1 << 30, n).astype(np.int64)
    probs = np.zeros(n, dtype=np.float32)
    at = rng.permutation(n)[:positive]
    probs[at] = rng.random(positive, dtype=np.float32) + 1e-3
    probs[rng.integers(0, n, 50)] = -1.0   # not positive: as good as zero
    sel, idx = capi.list_sample_weighted(to_dev(data, dev), to_dev(probs, dev), k, seed=5)
    w_sel, w_idx = O.list_sample_weighted(data, probs, k, seed=5)
    assert np.array_equal(idx.cpu().numpy(), w_idx)
    assert np.array_equal(sel.cpu().numpy(), w_sel)
    # closed form: every positive weight is picked, then the lowest positions without one
    n_pos = int((probs > 0).sum())
    assert set(w_idx[:n_pos].tolist()) == set(np.flatnonzero(probs > 0).tolist())
    assert np.array_equal(w_idx[n_pos:], np.flatnonzero(~(probs > 0))[:k - n_pos])


@pytest.mark.parametrize("n,k,distinct", [(60000, 700, 3), (20000, 5000, 1), (100000, 8192, 40)])
def test_list_weighted_keys_that_repeat_thousands_of_times(dev, n, k, distinct):
    """Replayed draws that are nearly all alike over equal weights: the class of the k-th key
    holds far more items than one sort takes, and positions decide inside a key."""
    rng = np.random.default_rng(n)
    data = np.arange(n, dtype=np.int64) * 7
    probs = np.full(n, 0.5, dtype=np.float32)
    values = rng.integers(1 << 30, 1 << 32, distinct, dtype=np.uint64).astype(np.uint32)
    replay = values[rng.integers(0, distinct, n)]
    sel, idx = capi.list_sample_weighted(to_dev(data, dev), to_dev(probs, dev), k,
                                         replay=to_dev(replay, dev))
    w_sel, w_idx = O.list_sample_weighted(data, probs, k, replay=replay)
    assert np.array_equal(idx.cpu().numpy(), w_idx)
    assert np.array_equal(sel.cpu().numpy(), w_sel)
    # closed form: equal weights, so the larger draw wins and the position breaks ties
    order = np.lexsort((np.arange(n), -(replay >> 8).astype(np.int64)))
    assert np.array_equal(w_idx, order[:k])


@pytest.mark.parametrize("case", range(16))
def test_list_weighted_on_seeded_random_shapes(dev, case):
    """n, k, the share of items without weight and the spread of the weights drawn from a seeded
    generator; half of the cases replay given draws."""
    rng = np.random.default_rng(500 + case)
    n = int(rng.choice([50, 3000, 70000, 400000]))
    k = int(min(n - 1, rng.choice([1, 10, 512, 3000, 8192])))
    data = rng.integers(0, 1 << 30, n).astype(np.int64)
    probs = (rng.random(n, dtype=np.float32) ** int(rng.choice([1, 4, 12]))).astype(np.float32)
    probs[rng.random(n) < rng.choice([0.0, 0.5, 0.97])] = 0.0
    idt = torch.int32 if case % 2 else torch.int64
    if case % 2:
        replay = u32_draws(n, case)
        sel, idx = capi.list_sample_weighted(to_dev(data, dev, idt), to_dev(probs, dev), k,
                                             replay=to_dev(replay, dev))
        w_sel, w_idx = O.list_sample_weighted(data, probs, k, replay=replay)
    else:
        sel, idx = capi.list_sample_weighted(to_dev(data, dev, idt), to_dev(probs, dev), k, seed=case)
        w_sel, w_idx = O.list_sample_weighted(data, probs, k, seed=case)
    assert np.array_equal(idx.cpu().numpy(), w_idx)
    assert np.array_equal(sel.cpu().numpy().astype(np.int64), w_sel)


def test_list_weighted_weights_at_any_alignment(dev):
    n, k = 100003, 300
    rng = np.random.default_rng(3)
    data = rng.integers(0, 1 << 30, n).astype(np.int64)
    probs = rng.random(n + 3, dtype=np.float32)
    t_probs = to_dev(probs, dev)
    for off in (1, 2, 3):
        sel, idx = capi.list_sample_weighted(to_dev(data, dev), t_probs[off:off + n], k, seed=2)
        assert np.array_equal(idx.cpu().numpy(),
                              O.list_sample_weighted(data, probs[off:off + n], k, seed=2)[1])


def test_list_weighted_replay(dev):
    n, k = 20000, 300
    rng = np.random.default_rng(8)
    data = np.arange(n, dtype=np.int64)
    probs = rng.random(n, dtype=np.float32) + 0.01
    replay = u32_draws(n, 6)
    sel, idx = capi.list_sample_weighted(to_dev(data, dev), to_dev(probs, dev), k, replay=to_dev(replay, dev))
    w_sel, w_idx = O.list_sample_weighted(data, probs, k, replay=replay)
    assert np.array_equal(idx.cpu().numpy(), w_idx)
    # closed form: argsort of the keys u^(1/w) computed in float64 (ties/rounding apart, the sets agree)
    u = ((replay >> 8).astype(np.float64) + 1) / 2.0 ** 24
    ref = np.argsort(-(np.log2(u) / probs.astype(np.float64)), kind="stable")[:k]
    assert len(set(ref.tolist()) ^ set(w_idx.tolist())) <= 2


def test_weighted_out_of_range_column_ids(dev):
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=14)
    probs = np.random.default_rng(1).random(indices.size, dtype=np.float32) + 0.1
    cols = np.array([3, -1, 1 << 10, 900, 1 << 20, 17], dtype=np.int64)
    got = _weighted_gpu(dev, indptr, indices, probs, cols, 4, seed=2)
    want = O.sample_weighted(indptr, indices, probs, cols, 4, seed=2)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


# ------------------------------------------------ with replacement (inverse CDF)
@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("fanout", [1, 7, 100])
def test_weighted_replace_matches_oracle(dev, fanout, fused, idt):
    n = 1 << 11
    indptr, indices = rmat_csc_np(n, 1 << 16, seed=21)
    rng = np.random.default_rng(fanout)
    probs = rng.random(indices.size).astype(np.float32)
    probs[rng.random(indices.size) < 0.1] = 0.0
    probs[rng.random(indices.size) < 0.02] = -1.0       # negative weights count as zero
    cols = rng.integers(0, n, size=300).astype(np.int64) if fused else None
    S = 300 if fused else n
    t_cols = None if cols is None else to_dev(cols, dev, idt)
    for replay in (None, u32_draws(S * fanout, seed=5)):
        got = capi.sample_weighted_replace(to_dev(indptr, dev), to_dev(indices, dev, idt),
                                           to_dev(probs, dev), t_cols, fanout, seed=11,
                                           replay=None if replay is None else to_dev(replay, dev),
                                           with_coo=True)
        want = O.sample_weighted_replace(indptr, indices, probs, cols, fanout, seed=11, replay=replay)
        nnz = int(want[0][-1])
        assert np.array_equal(got[0].cpu().numpy(), want[0])
        assert np.array_equal(got[1][:nnz].cpu().numpy().astype(np.int64), want[2])
        assert np.array_equal(got[2][:nnz].cpu().numpy(), want[3])
        assert np.array_equal(got[3][:nnz].cpu().numpy().astype(np.int64), want[1])
    # structure: fanout picks for every non-empty column, each inside the column, never an
    # edge of weight <= 0 while the column has a positive one
    c_of = np.arange(n) if cols is None else cols
    deg = np.diff(indptr)[c_of]
    assert np.array_equal(np.diff(want[0]), np.where(deg > 0, fanout, 0))
    sel = want[3]
    owner = want[1]
    assert ((sel >= indptr[c_of[owner]]) & (sel < indptr[c_of[owner] + 1])).all()
    has_pos = np.array([(probs[indptr[c]:indptr[c + 1]] > 0).any() for c in c_of])
    assert (probs[sel][has_pos[owner]] > 0).all()


def test_weighted_replace_hub_column_and_frequencies(dev):
    # one column of 20000 edges (313 scan chunks): frequencies follow the weights
    deg, k = 20000, 200000
    indptr = np.array([0, deg], dtype=np.int64)
    indices = np.arange(deg, dtype=np.int64)
    probs = np.ones(deg, dtype=np.float32)
    probs[:10] = 500.0                      # ten heavy edges share 5000 / 24990 of the mass
    got = capi.sample_weighted_replace(to_dev(indptr, dev), to_dev(indices, dev), to_dev(probs, dev),
                                       None, k, seed=3)
    want = O.sample_weighted_replace(indptr, indices, probs, None, k, seed=3)
    assert np.array_equal(got[1].cpu().numpy(), want[2])
    heavy = (want[2] < 10).sum()
    p = 5000.0 / 24990.0
    assert abs(heavy - k * p) < 6 * np.sqrt(k * p * (1 - p))
    counts = np.bincount(want[2][want[2] < 10], minlength=10)
    assert counts.min() > 0.8 * k * p / 10 and counts.max() < 1.2 * k * p / 10


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_weighted_replace_long_columns_block_by_block(dev, idt):
    # columns of several 2048-edge blocks between short ones, real-valued weights: the
    # blocks are scanned by separate waves and their sums added up in order, and every
    # pick must be the oracle's (same additions, same bits); lengths around the block size
    degs = [5, 2048, 0, 2049, 40000, 3, 4096, 4097, 1, 10000, 0, 70]
    indptr = np.concatenate([[0], np.cumsum(degs)]).astype(np.int64)
    rng = np.random.default_rng(8)
    indices = rng.integers(0, 1000, size=int(indptr[-1])).astype(np.int64)
    probs = rng.random(indices.size).astype(np.float32)
    probs[rng.random(indices.size) < 0.05] = -0.5
    k = 300
    for cols in (None, np.array([4, 9, 1, 4, 11, 3, 7, 2], dtype=np.int64)):
        S = len(degs) if cols is None else cols.size
        replay = u32_draws(S * k, seed=12)
        t_cols = None if cols is None else to_dev(cols, dev, idt)
        got = capi.sample_weighted_replace(to_dev(indptr, dev), to_dev(indices, dev, idt),
                                           to_dev(probs, dev), t_cols, k,
                                           replay=to_dev(replay, dev), with_coo=True)
        want = O.sample_weighted_replace(indptr, indices, probs, cols, k, replay=replay)
        nnz = int(want[0][-1])
        assert np.array_equal(got[0].cpu().numpy(), want[0])
        assert np.array_equal(got[2][:nnz].cpu().numpy(), want[3])
        assert np.array_equal(got[1][:nnz].cpu().numpy().astype(np.int64), want[2])
        assert np.array_equal(got[3][:nnz].cpu().numpy().astype(np.int64), want[1])


def test_graph_sampling_with_probs_replace(dev):
    import graph_sampling_amd as gs
    n = 1 << 10
    indptr, indices = rmat_csc_np(n, 1 << 14, seed=22)
    probs = np.random.default_rng(0).random(indices.size).astype(np.float32)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(to_dev(indptr, dev), to_dev(indices, dev))
    g._CAPI_SetData(to_dev(probs, dev))
    torch.ops.gs_ops._CAPI_SetSeed(99)
    sub = g._CAPI_SamplingWithProbs(0, to_dev(probs, dev).unsqueeze(1), 5, True, gs._CSC, gs._COO)
    want = O.sample_weighted_replace(indptr, indices, probs, None, 5, seed=99)
    row, col = sub._CAPI_GetBatchCOO()
    assert np.array_equal(row.cpu().numpy(), want[2]) and np.array_equal(col.cpu().numpy(), want[1])
    # the PASS sampler reads the picked edges' weights back in column order
    assert np.array_equal(sub._CAPI_GetData("col").cpu().numpy(), probs[want[3]])
    assert sub._CAPI_GetNumEdges() == want[2].size == 5 * int((np.diff(indptr) > 0).sum())
