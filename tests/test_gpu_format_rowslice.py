"""GPU parity: format conversion and row slicing vs the CPU oracle and closed forms."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import (graph_12col_4edge, graph_20x5, rmat_csc_np, row_slice_coo_closed_form,
                        to_dev)

pytestmark = pytest.mark.gpu

ID_DTYPES = [torch.int64, torch.int32]


def test_csc2coo_reference_vector(dev):
    # reference tests/test_format_transform.cc:7-28: col = repeat_interleave(arange(20), 5)
    indptr, _ = graph_20x5()
    col = capi.csc2coo(to_dev(indptr, dev), 100).cpu().numpy()
    assert np.array_equal(col, np.repeat(np.arange(20), 5))


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("seed", [1, 2])
def test_csc2coo_rmat(dev, seed, idt):
    indptr, indices = rmat_csc_np(1 << 13, 1 << 17, seed=seed)
    col = capi.csc2coo(to_dev(indptr, dev), indices.size, idt)
    assert col.dtype == idt
    col = col.cpu().numpy()
    assert np.array_equal(col, np.repeat(np.arange(indptr.size - 1), np.diff(indptr)))
    assert np.array_equal(col, O.csc2coo(indptr, indices.size))


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_csc2coo_runs_of_tiles_with_hubs_and_empty_columns(dev, idt):
    """From 2 x 4096 x 2048 edges on a workgroup walks through several 4096-edge tiles: hubs that
    cover many tiles, runs of more than 256 empty columns (several reads of the offsets for one
    tile), columns that start exactly on tile and span boundaries, empty columns at both ends."""
    rng = np.random.default_rng(3)
    deg = rng.integers(0, 60, size=700_000).astype(np.int64)
    deg[rng.integers(0, deg.size, size=40)] = rng.integers(20_000, 400_000, size=40)
    for at in rng.integers(0, deg.size - 2000, size=30):
        deg[at:at + rng.integers(257, 1500)] = 0
    deg[:300] = 0
    deg[-700:] = 0
    # make some columns start exactly on multiples of 4096 and of 3 x 4096
    ptr = np.concatenate([[0], np.cumsum(deg)])
    for c in rng.integers(1000, deg.size - 1000, size=200):
        pad = (-ptr[c]) % (4096 * (3 if c % 2 else 1))
        deg[c - 1] += pad
        ptr = np.concatenate([[0], np.cumsum(deg)])
    nnz = int(ptr[-1])
    assert nnz >= 3 * 4096 * 2048
    col = capi.csc2coo(to_dev(ptr, dev), nnz, idt)
    want = torch.repeat_interleave(torch.arange(deg.size, device=dev), to_dev(deg, dev))
    assert col.dtype == idt and torch.equal(col.long(), want)
    # the doubly-compressed form of the same: only the columns with edges are stored
    kept = np.flatnonzero(deg)
    d_ptr = np.concatenate([[0], np.cumsum(deg[kept])])
    d_col = capi.dcsc2coo(to_dev(d_ptr, dev), nnz, to_dev(kept, dev, idt))
    assert torch.equal(d_col.long(), want)


def test_coo2csc_reference_eids(dev):
    # reference tests/test_format_transform.cc:54-74: CSC -> CSR of the 12-column graph
    indptr, indices = graph_12col_4edge()
    col = np.repeat(np.arange(12), np.diff(indptr))          # [10,10,11,11]
    ip, val, perm = capi.coo2csc(to_dev(indices, dev), to_dev(col, dev), 12, False)
    assert np.array_equal(ip.cpu().numpy(), [0, 0, 2, 2] + [4] * 9)
    assert np.array_equal(val.cpu().numpy(), [10, 11, 10, 11])
    assert np.array_equal(perm.cpu().numpy(), [0, 2, 1, 3])


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("num_keys,E", [(1, 50), (7, 1000), (1 << 12, 1 << 17), (300000, 50000), (2_450_000, 200000)])
def test_coo2csc_unsorted_matches_stable_sort(dev, num_keys, E, idt):
    rng = np.random.default_rng(E)
    key = rng.integers(0, num_keys, size=E).astype(np.int64)
    value = rng.integers(0, 1 << (40 if idt == torch.int64 else 31), size=E).astype(np.int64)
    ip, val, perm = capi.coo2csc(to_dev(key, dev, idt), to_dev(value, dev, idt), num_keys, False)
    assert val.dtype == idt and perm.dtype == torch.int64
    want_perm = np.argsort(key, kind="stable")
    assert np.array_equal(perm.cpu().numpy(), want_perm)
    assert np.array_equal(val.cpu().numpy(), value[want_perm])
    want_ip = np.concatenate([[0], np.cumsum(np.bincount(key, minlength=num_keys))])
    assert np.array_equal(ip.cpu().numpy(), want_ip)
    o_ip, o_val, o_perm = O.coo2csc(key, value, num_keys, False)
    assert np.array_equal(o_ip, want_ip) and np.array_equal(o_perm, want_perm) and np.array_equal(o_val, value[want_perm])


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("num_keys,E", [(2, 1), (3, 2047), (255, 2048), (256, 2049), (257, 4096),
                                        (300, 4095), (70000, 4097), (5, 8191), (99, 8193),
                                        (65536, 6000), (65537, 6000), ((1 << 20) + 1, 70000),
                                        (10, 100000), (5000, 300000)])
def test_coo2csc_sizes_and_skew(dev, num_keys, E, idt):
    # edge counts around the sort tiles (2048 edges with 8-byte ids, 4096 with 4-byte ids) and
    # around a wave's share of a tile, key counts around the 8-bit digits (1, 2 and 3 passes),
    # and keys piled on few columns: the offsets of a 256-column workgroup are then searched in
    # more than the 4096 keys it can stage
    rng = np.random.default_rng(num_keys + E)
    key = (rng.random(E) ** 3 * num_keys).astype(np.int64)        # skewed towards the low keys
    key[rng.random(E) < 0.01] = num_keys - 1
    value = rng.integers(0, 1 << 31, size=E).astype(np.int64)
    ip, val, perm = capi.coo2csc(to_dev(key, dev, idt), to_dev(value, dev, idt), num_keys, False)
    want_perm = np.argsort(key, kind="stable")
    assert np.array_equal(perm.cpu().numpy(), want_perm)
    assert np.array_equal(val.cpu().numpy(), value[want_perm])
    want_ip = np.concatenate([[0], np.cumsum(np.bincount(key, minlength=num_keys))])
    assert np.array_equal(ip.cpu().numpy(), want_ip)
    # the same keys already sorted: offsets only
    ip2, _, _ = capi.coo2csc(to_dev(key[want_perm], dev, idt), to_dev(value[want_perm], dev, idt),
                             num_keys, True)
    assert np.array_equal(ip2.cpu().numpy(), want_ip)


def test_coo2csc_one_key_many_edges_keeps_input_order(dev):
    """Every edge under the same key (and under two keys at the ends of the digit range): the
    stable order is the input order, across waves, rounds and tiles."""
    E = 3 * 4096 + 77
    value = np.arange(E, dtype=np.int64)[::-1].copy()
    for keys in (np.zeros(E, dtype=np.int64), np.where(np.arange(E) % 3 == 0, 255, 0)):
        for idt in ID_DTYPES:
            ip, val, perm = capi.coo2csc(to_dev(keys, dev, idt), to_dev(value, dev, idt), 256, False)
            want = np.argsort(keys, kind="stable")
            assert np.array_equal(perm.cpu().numpy(), want)
            assert np.array_equal(val.cpu().numpy(), value[want])
            assert int(ip[-1]) == E


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_coo2csc_sorted(dev, idt):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 15, seed=3)
    col = np.repeat(np.arange(indptr.size - 1), np.diff(indptr))
    ip, val, perm = capi.coo2csc(to_dev(col, dev, idt), to_dev(indices, dev, idt), indptr.size - 1, True)
    assert perm is None
    assert np.array_equal(ip.cpu().numpy(), indptr)
    assert np.array_equal(val.cpu().numpy(), indices)


def test_row_slice_csc_reference_vector(dev):
    # reference tests/test_rowwise_slicing.cc:7-20: rows 0,5,..,95 of the 20x5 graph
    indptr, indices = graph_20x5()
    rows = np.arange(0, 100, 5, dtype=np.int64)
    got = capi.row_slice_csc(to_dev(indptr, dev), to_dev(indices, dev), to_dev(rows, dev), True)
    assert np.array_equal(got[0].cpu().numpy(), np.arange(21))
    assert np.array_equal(got[2].cpu().numpy(), np.arange(20))
    want = O.row_slice_csc(indptr, indices, rows, True)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("with_coo", [True, False])
@pytest.mark.parametrize("n_rows", [0, 1, 512, 4000])
def test_row_slice_csc_rmat(dev, with_coo, n_rows, idt):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=4)
    rows = np.random.default_rng(n_rows).permutation(1 << 12)[:n_rows].astype(np.int64)
    got = capi.row_slice_csc(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(rows, dev, idt),
                             with_coo)
    assert got[2].dtype == idt and got[3].dtype == torch.int64
    want = O.row_slice_csc(indptr, indices, rows, with_coo)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(g.cpu().numpy(), w)
    # closed form: mask + position lookup
    mask = np.isin(indices, rows)
    lut = np.full(1 << 12, -1)
    lut[rows] = np.arange(n_rows)
    assert np.array_equal(want[2], lut[indices[mask]])
    assert np.array_equal(want[3], np.nonzero(mask)[0])


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("n_rows", [300, 20000, 150000])
def test_row_slice_csc_many_edges(dev, n_rows, idt):
    """From 2^20 edges on the keys are tested by workgroups that stay, against a copy of the
    filter in LDS: the filter itself for few row ids, a folded one in front of it for many."""
    n = 1 << 18
    indptr, indices = rmat_csc_np(n, (1 << 21) + 777, seed=6)
    rows = np.random.default_rng(n_rows).permutation(n)[:n_rows].astype(np.int64)
    got = capi.row_slice_csc(to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(rows, dev, idt),
                             True)
    want = O.row_slice_csc(indptr, indices, rows, True)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)
    mask = np.isin(indices, rows)
    lut = np.full(n, -1)
    lut[rows] = np.arange(n_rows)
    assert np.array_equal(want[2], lut[indices[mask]])
    assert np.array_equal(want[3], np.nonzero(mask)[0])


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_row_slice_coo(dev, idt):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 16, seed=5)
    col = np.repeat(np.arange(indptr.size - 1), np.diff(indptr))
    ids = np.random.default_rng(0).permutation(1 << 12)[:512].astype(np.int64)
    got = capi.row_slice_coo(to_dev(indices, dev, idt), to_dev(col, dev, idt), to_dev(ids, dev, idt))
    want = O.row_slice_coo(indices, col, ids)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)
    # and against the closed form that does not go through the oracle, all three outputs
    for g, w in zip(got, row_slice_coo_closed_form(indices, col, ids)):
        assert np.array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("E", [0, 1, 63, 64, 65, 2047, 2048, 2049, 3 * 2048, 3 * 2048 + 64, 9001])
def test_row_slice_sizes_around_words_and_tiles(dev, E, idt):
    # the mark pass leaves one bit per edge in 64-edge words and counts per 2048-edge tile:
    # edge counts on both sides of those boundaries, kept edges everywhere / nowhere / mixed,
    # ids beyond 2^32 for the 64-bit type, duplicates among the row ids (largest position wins)
    rng = np.random.default_rng(E)
    big = (1 << 40) if idt == torch.int64 else 0
    key = rng.integers(0, 50, size=E).astype(np.int64) + big
    other = rng.integers(0, 1000, size=E).astype(np.int64)
    for ids in (np.arange(50, dtype=np.int64) + big,                       # everything kept
                np.array([77, 78], dtype=np.int64) + big,                  # nothing kept
                np.array([3, 17, 3, 42, 8, 17], dtype=np.int64) + big):    # mixed, duplicates
        got = capi.row_slice_coo(to_dev(key, dev, idt), to_dev(other, dev, idt), to_dev(ids, dev, idt))
        want = O.row_slice_coo(key, other, ids)
        for g, w, c in zip(got, want, row_slice_coo_closed_form(key, other, ids)):
            assert np.array_equal(g.cpu().numpy(), w)
            assert np.array_equal(w, c)
        # the same edges as a CSC of 7 columns with empty ones in between
        cuts = np.sort(rng.integers(0, E + 1, size=6))
        indptr = np.concatenate([[0], cuts, [E]]).astype(np.int64)
        got = capi.row_slice_csc(to_dev(indptr, dev), to_dev(key, dev, idt), to_dev(ids, dev, idt), True)
        want = O.row_slice_csc(indptr, key, ids, True)
        for g, w in zip(got, want):
            assert np.array_equal(g.cpu().numpy(), w)
        # membership filter: both ends kept as they are
        got = capi.coo_filter(to_dev(key, dev, idt), to_dev(key, dev, idt), to_dev(other, dev, idt),
                              to_dev(ids, dev, idt))
        mask = np.isin(key, ids)
        assert np.array_equal(got[0].cpu().numpy(), key[mask])
        assert np.array_equal(got[1].cpu().numpy(), other[mask])
        assert np.array_equal(got[3].cpu().numpy(), np.nonzero(mask)[0])
