"""GPU parity: column slicing and uniform sampling through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import graph_20x5, rmat_csc_np, to_dev, u32_draws

pytestmark = pytest.mark.gpu

ID_DTYPES = [torch.int64, torch.int32]


def _slice_gpu(indptr, indices, cols, with_coo):
    sub_indptr = capi.slice_count(indptr, cols)
    nnz = int(sub_indptr[-1].item())
    sub_indices, select_index, coo_col = capi.slice_fill(indptr, indices, cols, sub_indptr, nnz, with_coo)
    return sub_indptr, coo_col, sub_indices, select_index


def _cmp(got, want):
    for g, w in zip(got, want):
        if w is None:
            assert g is None
            continue
        g = g.cpu().numpy().astype(np.int64)
        assert g.shape == w.shape, (g.shape, w.shape)
        assert np.array_equal(g, w)


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_slice_reference_vector(dev, idt):
    # reference tests/test_colwise_slicing.cc:7-20
    indptr, indices = graph_20x5()
    cols = np.arange(3, dtype=np.int64)
    got = _slice_gpu(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt), True)
    assert np.array_equal(got[0].cpu().numpy(), np.arange(4) * 5)
    assert np.array_equal(got[2].cpu().numpy(), np.arange(15))
    _cmp(got, O.slice_columns(indptr, indices, cols, True))


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("with_coo", [True, False])
@pytest.mark.parametrize("S", [0, 1, 7, 513, 5000])
def test_slice_rmat(dev, idt, with_coo, S):
    indptr, indices = rmat_csc_np(1 << 13, 1 << 17, seed=3)
    rng = np.random.default_rng(S)
    cols = rng.integers(0, indptr.size - 1, size=S).astype(np.int64)  # duplicates allowed
    if S > 3:
        cols[1] = int(np.argmax(np.diff(indptr)))  # the hub column
        cols[2] = int(np.argmin(np.diff(indptr)))  # an empty / tiny column
    got = _slice_gpu(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt), with_coo)
    _cmp(got, O.slice_columns(indptr, indices, cols, with_coo))


def test_slice_many_empty_columns(dev):
    # more rows than the LDS stage holds inside one 2048-edge tile
    deg = np.zeros(6000, dtype=np.int64)
    deg[::7] = 1
    deg[5999] = 3000
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = np.arange(indptr[-1], dtype=np.int64)[::-1].copy()
    cols = np.arange(6000, dtype=np.int64)
    got = _slice_gpu(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev), True)
    _cmp(got, O.slice_columns(indptr, indices, cols, True))


ALGOS = [O.ALGO_AUTO, O.ALGO_RESERVOIR]


def _sample_gpu(indptr, indices, cols, k, replace, seed=0, replay=None, replay_ptr=None, with_coo=True,
                algo=O.ALGO_AUTO):
    sub_indptr, si, sel, coo = capi.sample_uniform(indptr, indices, cols, k, replace, seed=seed,
                                                   replay=replay, replay_ptr=replay_ptr,
                                                   with_coo=with_coo, algo=algo)
    nnz = int(sub_indptr[-1].item())
    return sub_indptr, None if coo is None else coo[:nnz], si[:nnz], sel[:nnz]


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_sample_identity_reference_vector(dev, idt):
    # reference tests/test_colwise_sampling.cc:7-20: fanout 6 >= degree 5 -> identity
    indptr, indices = graph_20x5()
    got = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev, idt), None, 6, False)
    assert np.array_equal(got[0].cpu().numpy(), indptr)
    assert np.array_equal(got[2].cpu().numpy(), indices)


@pytest.mark.parametrize("fanout", [6, 4])
def test_sample_replace_reference_counts(dev, fanout):
    # reference tests/test_colwise_sampling.cc:22-53
    indptr, indices = graph_20x5()
    got = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev), None, fanout, True)
    assert np.array_equal(got[0].cpu().numpy(), np.arange(21) * fanout)
    idx = got[2].cpu().numpy()
    assert idx.size == 20 * fanout
    assert np.unique(idx).size <= 100
    _cmp(got, O.sample_uniform(indptr, indices, None, fanout, True, seed=0))


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("k", [1, 5, 15, 16, 17, 33, 64, 65, 1000])
@pytest.mark.parametrize("fused", [True, False])
def test_sample_free_running_matches_oracle(dev, idt, replace, k, fused, algo):
    """Philox is integer-only, so even free-running draws match the oracle bit for bit."""
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=5)  # avg deg 32, hubs of several thousand
    if fused:
        rng = np.random.default_rng(k)
        cols = rng.integers(0, indptr.size - 1, size=3000).astype(np.int64)
        cols[:8] = np.argsort(np.diff(indptr))[-8:]  # the hub columns
        dcols = to_dev(cols, dev, idt)
    else:
        cols, dcols = None, None
    got = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev, idt), dcols, k, replace, seed=1234 + k,
                      algo=algo)
    want = O.sample_uniform(indptr, indices, cols, k, replace, seed=1234 + k, algo=algo)
    _cmp(got, want)


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("k", [3, 15, 900])
def test_sample_replay_matches_oracle(dev, replace, k, algo):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=6)
    cols = np.random.default_rng(1).integers(0, indptr.size - 1, size=2000).astype(np.int64)
    cols[:4] = np.argsort(np.diff(indptr))[-4:]
    _, replay_ptr = O.sample_count(indptr, cols, k, replace, want_replay_ptr=True, algo=algo)
    replay = u32_draws(int(replay_ptr[-1]), seed=k)
    want = O.sample_uniform(indptr, indices, cols, k, replace, replay=replay, algo=algo)
    got = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev), k, replace,
                      replay=to_dev(replay, dev), replay_ptr=to_dev(replay_ptr, dev), algo=algo)
    _cmp(got, want)


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("k", [5, 1000])
def test_sample_star_hub_many_chunks(dev, k, algo):
    # one column of degree 300k (74 chunks of 4096 draws) among small ones
    degs = np.array([3, 300000, 0, 17, 2000, 70000], dtype=np.int64)
    indptr = np.concatenate([[0], np.cumsum(degs)]).astype(np.int64)
    indices = np.random.default_rng(0).integers(0, 1 << 20, size=int(indptr[-1])).astype(np.int64)
    cols = np.array([1, 0, 5, 1, 2, 3, 4, 5], dtype=np.int64)
    got = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev), k, False, seed=77,
                      algo=algo)
    _cmp(got, O.sample_uniform(indptr, indices, cols, k, False, seed=77, algo=algo))


@pytest.mark.parametrize("algo", ALGOS)
def test_sample_structural_invariants(dev, algo):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=7)
    cols = np.random.default_rng(2).integers(0, indptr.size - 1, size=4096).astype(np.int64)
    k = 10
    sub_indptr, _, si, sel = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev),
                                         k, False, seed=99, with_coo=False, algo=algo)
    sub_indptr, si, sel = sub_indptr.cpu().numpy(), si.cpu().numpy(), sel.cpu().numpy()
    deg = indptr[cols + 1] - indptr[cols]
    assert np.array_equal(np.diff(sub_indptr), np.minimum(deg, k))
    assert np.array_equal(indices[sel], si)
    for r in range(cols.size):
        s = sel[sub_indptr[r]:sub_indptr[r + 1]]
        assert np.all((s >= indptr[cols[r]]) & (s < indptr[cols[r] + 1]))
        assert np.unique(s).size == s.size


@pytest.mark.parametrize("algo", ALGOS)
def test_sample_chi_square_inclusion(dev, algo):
    """Each edge of a degree-d column is kept with probability k/d (both algorithms)."""
    d, k, trials = 40, 8, 4000
    indptr = np.array([0, d], dtype=np.int64)  # one column sampled `trials` times
    indices = np.arange(d, dtype=np.int64)
    cols = np.zeros(trials, dtype=np.int64)  # duplicate seeds get independent draws (row-keyed)
    _, _, si, _ = _sample_gpu(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev), k, False,
                              seed=2024, with_coo=False, algo=algo)
    counts = np.bincount(si.cpu().numpy(), minlength=d).astype(np.float64)
    expect = trials * k / d
    # positions are exchangeable up to the (negligible) dependence inside a draw; 39 dof
    chi2 = ((counts - expect) ** 2 / (expect * (1 - k / d))).sum()
    assert chi2 < 39 + 5 * np.sqrt(2 * 39), chi2


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_one_keepdim(dev, idt):
    indptr, indices = rmat_csc_np(1 << 10, 1 << 13, seed=8)
    cols = np.arange(1 << 10, dtype=np.int64)
    got = capi.sample_one_keepdim(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt),
                                  seed=5)
    want = O.sample_one_keepdim(indptr, indices, cols, seed=5)
    assert (np.diff(indptr) == 0).any()  # the -1 branch is exercised
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy().astype(np.int64), w)
    replay = u32_draws(cols.size, 3)
    got = capi.sample_one_keepdim(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt),
                                  replay=to_dev(replay, dev))
    want = O.sample_one_keepdim(indptr, indices, cols, replay=replay)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy().astype(np.int64), w)


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_out_of_range_column_ids_are_empty_columns(dev, idt):
    """A stray id (-1 from a dead-end step, or >= num_cols) is an empty column, never dereferenced."""
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=12)
    n = 1 << 10
    cols = np.random.default_rng(0).integers(0, n, size=600).astype(np.int64)
    cols[::7] = -1
    cols[3::11] = n
    cols[5::13] = n + 12345
    d_ip, d_ix, d_cols = to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt)
    _cmp(_slice_gpu(d_ip, d_ix, d_cols, True), O.slice_columns(indptr, indices, cols, True))
    for algo in ALGOS:
        for replace in (False, True):
            got = _sample_gpu(d_ip, d_ix, d_cols, 6, replace, seed=3, algo=algo)
            _cmp(got, O.sample_uniform(indptr, indices, cols, 6, replace, seed=3, algo=algo))
    got = capi.sample_one_keepdim(d_ip, d_ix, d_cols, seed=4)
    want = O.sample_one_keepdim(indptr, indices, cols, seed=4)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy().astype(np.int64), w)
    assert (want[1][::7] == -1).all()
