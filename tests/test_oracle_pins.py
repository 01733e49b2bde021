"""Pins the CPU oracle (no GPU): the reference's own test vectors, closed forms that a wrong
index / sign / dropped term would break, brute force on tiny inputs, published RNG vectors."""
import collections
import itertools
import json
import math
import os

import numpy as np
import pytest

from oracle import oracle as O
from tests.util import (graph_12col_4edge, graph_20x5, rmat_csc_np, row_slice_coo_closed_form,
                        u32_draws)

HERE = os.path.dirname(os.path.abspath(__file__))
REF = json.load(open(os.path.join(HERE, "golden", "reference_vectors.json")))
GOLD = np.load(os.path.join(HERE, "golden", "replay_small.npz"))


# ------------------------------------------------------------------ RNG / keys
def test_philox_known_answer_vectors():
    for kat in REF["philox4x32_10_kat"]:
        assert O.philox4x32_10(kat["ctr"], kat["key"]).tolist() == kat["out"]


def test_draw_is_philox_keyed_by_seed_row_idx():
    seed, tag, row, idx = 0x1234567890ABCDEF, 3, (5 << 32) | 77, 1002
    q = idx >> 2
    block = O.philox4x32_10([q & 0xFFFFFFFF, row & 0xFFFFFFFF, row >> 32, tag | ((q >> 32) << 8)],
                            [seed & 0xFFFFFFFF, seed >> 32])
    assert O.draw(seed, tag, row, idx) == int(block[idx & 3])
    # different rows / tags / seeds give different streams
    assert len({O.draw(1, 1, r, 0) for r in range(50)}) == 50
    assert O.draw(1, 1, 0, 0) != O.draw(1, 2, 0, 0) != O.draw(2, 1, 0, 0)


def test_log2_u24_against_libm():
    xs = np.concatenate([[0, 255, 256, 1 << 31, 0xFFFFFFFF], u32_draws(20000, 1)]).astype(np.uint64)
    for x in xs[:3000]:
        m = (int(x) >> 8) + 1
        want = math.log2(m / 2.0 ** 24)
        assert abs(O.log2_u24(int(x)) - want) <= 3e-7 * max(1.0, abs(want))
    assert O.log2_u24(0xFFFFFFFF) == 0.0
    assert O.ares_key(123, 0.0) == -math.inf and O.ares_key(123, -1.0) == -math.inf
    # monotone in u (the order A-Res needs)
    ks = [O.log2_u24(int(v) << 8) for v in range(1, 5000)]
    assert all(a <= b for a, b in zip(ks, ks[1:]))


# -------------------------------------------------------------------- slicing
def test_slice_reference_vector():
    g = REF["graph_20x5"]
    v = REF["colwise_slicing_test1"]
    sp, coo, si, sel = O.slice_columns(g["indptr"], g["indices"], v["cols"])
    assert sp.tolist() == v["indptr"] and si.tolist() == v["indices"]
    assert coo.tolist() == np.repeat(np.arange(3), 5).tolist() and sel.tolist() == list(range(15))


def test_slice_closed_form():
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=1)
    cols = np.random.default_rng(0).integers(0, 1 << 10, 300)  # duplicates allowed, order kept
    sp, coo, si, sel = O.slice_columns(indptr, indices, cols)
    ranges = [np.arange(indptr[c], indptr[c + 1]) for c in cols]
    assert np.array_equal(sel, np.concatenate(ranges))
    assert np.array_equal(si, indices[sel])
    assert np.array_equal(coo, np.repeat(np.arange(cols.size), [r.size for r in ranges]))
    assert np.array_equal(sp, np.concatenate([[0], np.cumsum([r.size for r in ranges])]))


# ------------------------------------------------------------------- sampling
def test_sampling_reference_vectors():
    g = REF["graph_20x5"]
    for algo in (O.ALGO_AUTO, O.ALGO_RESERVOIR):
        v = REF["colwise_sampling_test1"]
        sp, _, si, _ = O.sample_uniform(g["indptr"], g["indices"], None, v["fanout"], False, algo=algo)
        assert sp.tolist() == v["indptr"] and si.tolist() == v["indices"]
    for name in ("colwise_sampling_test2", "colwise_sampling_test3"):
        v = REF[name]
        sp, _, si, _ = O.sample_uniform(g["indptr"], g["indices"], None, v["fanout"], True)
        assert sp.tolist() == v["indptr"] and si.size == 20 * v["fanout"]
        assert np.unique(si).size <= v["max_unique"] and not np.array_equal(si, g["indices"][:si.size])
        # every sample of column c comes from column c
        assert np.array_equal(si // 5, np.repeat(np.arange(20), v["fanout"]))


def _algorithm_r(deg, k, draws):
    """Textbook sequential Algorithm R (Vitter 1985) given the draws for idx = k..deg-1."""
    slot = list(range(k))
    for idx in range(k, deg):
        num = int(draws[idx - k]) % (idx + 1)
        if num < k:
            slot[num] = idx
    return slot


def _floyd(deg, k, draws):
    """Bentley & Floyd 1987, given the draws for steps 0..k-1; insertion order."""
    chosen = []
    for i in range(k):
        j = deg - k + i
        t = int(draws[i]) % (j + 1)
        chosen.append(j if t in chosen else t)
    return chosen


@pytest.mark.parametrize("algo,model", [(O.ALGO_RESERVOIR, _algorithm_r), (O.ALGO_AUTO, _floyd)])
def test_sampling_replay_equals_textbook_algorithm(algo, model):
    indptr, indices = rmat_csc_np(1 << 9, 1 << 13, seed=2)
    cols = np.random.default_rng(1).integers(0, 1 << 9, 200)
    k = 7
    sp, rp = O.sample_count(indptr, cols, k, False, want_replay_ptr=True, algo=algo)
    draws = u32_draws(int(rp[-1]), 3)
    _, coo, si, sel = O.sample_uniform(indptr, indices, cols, k, False, replay=draws, algo=algo)
    for r, c in enumerate(cols):
        deg = indptr[c + 1] - indptr[c]
        got = sel[sp[r]:sp[r + 1]] - indptr[c]
        if deg <= k:
            assert got.tolist() == list(range(deg))
        else:
            assert got.tolist() == model(int(deg), k, draws[rp[r]:rp[r + 1]])
    assert np.array_equal(si, indices[sel])
    assert np.array_equal(coo, np.repeat(np.arange(cols.size), np.diff(sp)))


def test_floyd_is_uniform_over_subsets_by_enumeration():
    n, k = 6, 3
    indptr, indices = np.array([0, n]), np.arange(n)
    cnt = collections.Counter()
    for d in itertools.product(*[range(n - k + 1 + i) for i in range(k)]):
        _, _, si, _ = O.sample_uniform(indptr, indices, None, k, False, replay=np.array(d, dtype=np.uint32))
        cnt[tuple(sorted(si))] += 1
    assert len(cnt) == math.comb(n, k) and len(set(cnt.values())) == 1


def test_reservoir_is_uniform_over_subsets_by_enumeration():
    n, k = 5, 2
    indptr, indices = np.array([0, n]), np.arange(n)
    cnt = collections.Counter()
    for d in itertools.product(*[range(idx + 1) for idx in range(k, n)]):
        _, _, si, _ = O.sample_uniform(indptr, indices, None, k, False, algo=O.ALGO_RESERVOIR,
                                       replay=np.array(d, dtype=np.uint32))
        cnt[tuple(sorted(si))] += 1
    assert len(cnt) == math.comb(n, k) and len(set(cnt.values())) == 1


def test_one_keepdim_closed_form():
    indptr, indices = rmat_csc_np(1 << 9, 1 << 11, seed=3)
    cols = np.arange(1 << 9)
    replay = u32_draws(cols.size, 2)
    sp, si, sel = O.sample_one_keepdim(indptr, indices, cols, replay=replay)
    deg = np.diff(indptr)
    want_sel = np.where(deg > 0, indptr[:-1] + replay % np.maximum(deg, 1), -1)
    assert np.array_equal(sel, want_sel) and np.array_equal(sp, np.arange(cols.size + 1))
    assert np.array_equal(si, np.where(deg > 0, indices[np.maximum(want_sel, 0)], -1))
    assert (deg == 0).any()


def test_weighted_closed_form_and_special_cases():
    indptr, indices = rmat_csc_np(1 << 8, 1 << 12, seed=4)
    k = 5
    rng = np.random.default_rng(5)
    probs = (1.0 - rng.random(indices.size)).astype(np.float32)
    rp = O.weighted_replay_ptr(indptr, None, k)
    draws = u32_draws(int(rp[-1]), 6)
    sp, _, si, sel = O.sample_weighted(indptr, indices, probs, None, k, replay=draws)
    for c in range(indptr.size - 1):
        deg = indptr[c + 1] - indptr[c]
        got = sel[sp[c]:sp[c + 1]] - indptr[c]
        if deg <= k:
            assert got.tolist() == list(range(deg))
            continue
        u = ((draws[rp[c]:rp[c + 1]] >> 8).astype(np.float64) + 1) / 2.0 ** 24
        key = u ** (1.0 / probs[indptr[c]:indptr[c + 1]].astype(np.float64))  # the reference's key
        order = np.argsort(-key, kind="stable")
        # same set and order wherever float64 separates the keys clearly
        gaps = np.abs(np.diff(np.sort(np.log2(key))[::-1][:k + 1]))
        if gaps.min() > 1e-5:
            assert got.tolist() == order[:k].tolist()
    # equal weights: order of u alone; a zero weight is never picked while positives remain
    probs2 = np.ones(10, dtype=np.float32)
    probs2[3] = 0.0
    dr = u32_draws(10, 9)
    _, _, si2, _ = O.sample_weighted(np.array([0, 10]), np.arange(10), probs2, None, 4, replay=dr)
    u = (dr >> 8).astype(np.int64)
    u[3] = -1
    assert si2.tolist() == np.argsort(-u, kind="stable")[:4].tolist()


def test_weighted_replace_closed_form_and_special_cases():
    # integer weights: every order of float additions gives the same prefix sums, so the
    # picks must equal a plain cumsum + searchsorted; 150 edges = three scan chunks
    rng = np.random.default_rng(4)
    deg, k = 150, 4000
    indptr = np.array([0, 0, deg], dtype=np.int64)               # column 0 is empty
    indices = rng.permutation(1000)[:deg].astype(np.int64)
    w = rng.integers(0, 6, size=deg).astype(np.float32)
    w[7] = -3.0                                                   # counts as zero
    draws = u32_draws(2 * k, seed=9)
    ptr, col, idx, sel = O.sample_weighted_replace(indptr, indices, w, None, k, replay=draws)
    assert ptr.tolist() == [0, 0, k] and (col == 1).all()
    cdf = np.cumsum(np.maximum(w, 0), dtype=np.float32)
    u = ((draws[k:] >> 8).astype(np.float32) + np.float32(1)) * np.float32(2.0 ** -24)
    want = np.minimum(np.searchsorted(cdf, u * cdf[-1], side="right"), deg - 1)
    assert np.array_equal(sel, want) and np.array_equal(idx, indices[want])
    assert (w[sel] > 0).all()
    # frequencies follow the weights (chi-square over the edges with positive weight)
    pos = np.flatnonzero(w > 0)
    obs = np.bincount(sel, minlength=deg)[pos]
    exp = k * w[pos] / w[pos].sum()
    assert ((obs - exp) ** 2 / exp).sum() < pos.size + 6 * math.sqrt(2 * pos.size)
    # one edge carries all the weight: it is every pick
    one = np.zeros(deg, dtype=np.float32)
    one[42] = 2.5
    assert (O.sample_weighted_replace(indptr, indices, one, None, 50, seed=1)[3] == 42).all()
    # a column of several 2048-edge blocks (their sums are added up block by block): with
    # integer weights the order of additions cannot matter, so plain cumsum + searchsorted
    # must give the same picks
    big = 2048 * 3 + 700
    bptr = np.array([0, big], dtype=np.int64)
    bind = np.arange(big, dtype=np.int64)
    bw = rng.integers(0, 4, size=big).astype(np.float32)
    bdraws = u32_draws(5000, seed=10)
    bsel = O.sample_weighted_replace(bptr, bind, bw, None, 5000, replay=bdraws)[3]
    bcdf = np.cumsum(bw, dtype=np.float64).astype(np.float32)     # exact: integers below 2^24
    bu = ((bdraws >> 8).astype(np.float32) + np.float32(1)) * np.float32(2.0 ** -24)
    assert np.array_equal(bsel, np.minimum(np.searchsorted(bcdf, bu * bcdf[-1], side="right"),
                                           big - 1))
    # the Philox draw of pick j of row r is draw(seed, tag 2, r, j)
    _, _, _, a = O.sample_weighted_replace(indptr, indices, w, None, 8, seed=77)
    d = np.array([O.draw(77, 2, 1, j) for j in range(8)], dtype=np.uint32)
    _, _, _, b = O.sample_weighted_replace(indptr, indices, w, None, 8,
                                           replay=np.concatenate([np.zeros(8, np.uint32), d]))
    assert np.array_equal(a, b)


def test_list_sampling_reference_and_closed_form():
    v = REF["list_sampling"]
    data = np.arange(v["n"])
    sel, idx = O.list_sample_uniform(data, v["identity_k"], False)
    assert np.array_equal(sel, data) and np.array_equal(idx, data)
    sel, _ = O.list_sample_uniform(data, v["replace_k"], True, seed=1)
    assert sel.size == v["replace_k"] and np.unique(sel).size <= v["n"] and not np.array_equal(sel[:1000], data)
    sel, _ = O.list_sample_uniform(data, v["distinct_k"], False, seed=1)
    assert np.unique(sel).size == v["distinct_k"]
    dr = u32_draws(1000 - 100, 3)
    _, idx = O.list_sample_uniform(data, 100, False, replay=dr)
    assert idx.tolist() == _algorithm_r(1000, 100, dr)
    # weighted: identity when n <= k, zero weights last, closed form on the keys
    sel, idx = O.list_sample_weighted(data[:5], np.ones(5, np.float32), 9)
    assert np.array_equal(idx, np.arange(5))
    probs = np.random.default_rng(4).random(1000).astype(np.float32)
    dr = u32_draws(1000, 8)
    _, idx = O.list_sample_weighted(data, probs, 50, replay=dr)
    u = ((dr >> 8).astype(np.float64) + 1) / 2.0 ** 24
    ref = np.argsort(-(np.log2(u) / probs.astype(np.float64)), kind="stable")[:50]
    assert len(set(ref.tolist()) ^ set(idx.tolist())) <= 2


# ------------------------------------------------------------- unique / relabel
def test_relabel_reference_vectors():
    # tests/test_relabel.cc:7-26: slicing columns 1..3 with relabel maps rows 5..19 to 0..14
    g = REF["graph_20x5"]
    v = REF["slicing_relabel_test1"]
    _, _, si, _ = O.slice_columns(g["indptr"], g["indices"], v["cols"])
    frontier, (rel,) = O.relabel([si], [si])
    assert frontier.size == v["num_rows"] and rel.tolist() == v["indices"]
    # tests/test_format_transform.cc:25,49: AllValidNode = unique(cat(col_ids, rows))
    assert O.unique(np.concatenate([np.arange(20), np.arange(100)])).tolist() == list(range(100))
    assert O.unique(np.concatenate([np.arange(21), np.arange(2, 102)])).tolist() == list(range(102))


def test_unique_closed_form():
    x = np.random.default_rng(0).integers(0, 3000, 20000) * 977 % 10007
    u, first = np.unique(x, return_index=True)
    want = u[np.argsort(first, kind="stable")]
    assert np.array_equal(O.unique(x), want)
    frontier, (rel, miss) = O.relabel([x[:5000], x[5000:]], [x, np.array([10**9, int(x[0])])])
    assert np.array_equal(frontier, want) and np.array_equal(frontier[rel], x)
    assert miss.tolist() == [-1, 0]


# ----------------------------------------------------------------------- walks
def test_walk_reference_vectors():
    v = REF["hetero_walk_one_path"]
    rel = {"follow": 0, "view": 1}
    ips = [v["follow"]["indptr"], v["view"]["indptr"]]
    ixs = [v["follow"]["indices"], v["view"]["indices"]]
    tr = O.metapath_walk(ips, ixs, [rel[m] for m in v["metapath"]], v["seeds"], seed=5)
    assert tr.tolist() == v["trace_step_major"]
    v = REF["hetero_walk_multi_path"]
    ips = [v["follow"]["indptr"], v["view"]["indptr"]]
    ixs = [v["follow"]["indices"], v["view"]["indices"]]
    mp = [rel[m] for m in v["metapath"]]
    tr = O.metapath_walk(ips, ixs, mp, v["seeds"], seed=5).reshape(4, 5)
    for w in range(5):
        for t in range(3):
            s, d = tr[t, w], tr[t + 1, w]
            if d != -1:
                assert d in ixs[mp[t]][ips[mp[t]][s]:ips[mp[t]][s + 1]]
            if s == -1:
                assert d == -1


def test_walk_closed_form():
    indptr, indices = rmat_csc_np(1 << 9, 1 << 12, seed=6)
    n, L = 400, 5
    seeds = np.random.default_rng(2).integers(0, 1 << 9, n)
    replay = u32_draws(n * L, 4)
    tr = O.random_walk(indptr, indices, seeds, L, replay=replay).reshape(L + 1, n)
    assert np.array_equal(tr[0], seeds)
    for t in range(L):
        cur = tr[t]
        deg = np.where(cur >= 0, indptr[np.maximum(cur, 0) + 1] - indptr[np.maximum(cur, 0)], 0)
        pos = indptr[np.maximum(cur, 0)] + replay[t * n:(t + 1) * n] % np.maximum(deg, 1)
        want = np.where(deg > 0, indices[np.minimum(pos, indices.size - 1)], -1)
        assert np.array_equal(tr[t + 1], want)


# ---------------------------------------------------------- segment ops / SDDMM
def test_graph_compute_reference_vectors():
    g20, g12 = REF["graph_20x5"], REF["graph_12col"]
    ones = np.ones(100, np.float32)
    assert O.segment_sum(g20["indptr"], None, None, ones, 1, 20).tolist() == REF["graph_sum_test1"]["expected"]
    assert O.segment_sum(g20["indptr"], None, None, REF["graph_sum_test2"]["data"], 1, 20).tolist() == REF["graph_sum_test2"]["expected"]
    assert O.segment_sum(g20["indptr"], None, None, ones, 2, 20).tolist() == REF["graph_sum_test3"]["expected"]
    assert O.segment_sum(g20["indptr"], None, None, REF["graph_sum_test4"]["data"], 2, 20).tolist() == REF["graph_sum_test4"]["expected"]
    # row sums: CSR built by the stable COO->CSC conversion, data reached through e_ids
    col = O.csc2coo(g12["indptr"], 4)
    ip, val, perm = O.coo2csc(g12["indices"], col, 12, False)
    v = REF["graph_sum_test5"]
    assert O.segment_sum(ip, perm, None, v["data"], 1, 12).tolist() == v["expected"]
    assert O.coo_sum(g12["indices"], None, v["data"], 1, 12).tolist() == v["expected"]
    # Divide(divisor, axis 0, CSC) = SDDMM div with lhs = edge data, rhs = per-column divisor
    div = np.array(REF["graph_div_test2"]["divisor"], np.float32)
    out = O.sddmm_csc("div", g20["indptr"], g20["indices"], None, None, ones, div, 1, 2)
    np.testing.assert_allclose(out[:, 0], np.repeat(1 / div, 5), rtol=1e-6)
    # normalise rows of the 2-column slice
    v = REF["graph_normalize_test4"]
    rs = O.segment_sum(ip, perm, None, v["data"], 1, 12)
    out = O.sddmm_csc("div", ip, val, perm, None, np.array(v["data"], np.float32), rs, 1, 2)
    np.testing.assert_allclose(out[:, 0], v["expected"], rtol=1e-6)
    np.testing.assert_allclose(O.segment_normalize(ip, perm, v["data"]), v["expected"], rtol=1e-6)


def test_segment_ops_closed_form():
    indptr, indices = rmat_csc_np(1 << 9, 1 << 13, seed=7)
    rng = np.random.default_rng(3)
    data = rng.random(indices.size).astype(np.float32)
    col = np.repeat(np.arange(1 << 9), np.diff(indptr))
    for powk in (1, 2, 3):
        want = np.bincount(col, weights=data.astype(np.float64) ** powk, minlength=1 << 9)
        np.testing.assert_allclose(O.segment_sum(indptr, None, None, data, powk, 1 << 9), want, rtol=1e-5)
        np.testing.assert_allclose(O.coo_sum(indices, None, data, powk, 1 << 9),
                                   np.bincount(indices, weights=data.astype(np.float64) ** powk, minlength=1 << 9), rtol=1e-5)
    emap = rng.permutation(indices.size)
    nmap = rng.permutation(1 << 9)
    got = O.segment_sum(indptr, emap, nmap, data, 1, 1 << 9)
    want = np.zeros(1 << 9)
    want[nmap] = np.bincount(col, weights=data[emap].astype(np.float64), minlength=1 << 9)
    np.testing.assert_allclose(got, want, rtol=1e-5)
    divisor = rng.random(1 << 9).astype(np.float32) + 0.5
    od, osum = O.e_div_u_sum(indices, col, data, divisor, 1 << 9)
    assert np.array_equal(od, data / divisor[indices])
    np.testing.assert_allclose(osum, np.bincount(col, weights=od.astype(np.float64), minlength=1 << 9), rtol=1e-5)


def test_sddmm_reference_vectors_and_bcast():
    n = REF["sddmm_add_test1"]["n"]
    r = np.arange(n)
    f = np.arange(n, dtype=np.float32)
    assert np.array_equal(O.sddmm_coo("add", r, r, None, f, f, 0, 2)[:, 0], 2 * f)
    g = REF["graph_20x5"]
    rhs = np.arange(REF["sddmm_add_test2"]["rhs_n"], dtype=np.float32)
    col = O.csc2coo(g["indptr"], 100)
    want = f + np.repeat(rhs, 5)
    assert np.array_equal(O.sddmm_coo("add", g["indices"], col, None, f, rhs, 0, 2)[:, 0], want)
    assert np.array_equal(O.sddmm_csc("add", g["indptr"], g["indices"], None, None, f, rhs, 0, 2)[:, 0], want)
    # the worked example of the reference's bcast.h:20-30
    b = O.calc_bcast("add", (1, 1, 3), (1, 5, 1))
    assert b["lhs_off"].tolist() == [0, 1, 2] * 5 and b["rhs_off"].tolist() == sorted(list(range(5)) * 3)
    assert (b["out_len"], b["lhs_len"], b["rhs_len"], b["reduce_size"]) == (15, 3, 5, 1)
    b = O.calc_bcast("dot", (1, 3, 5), (1, 3, 5))
    assert (b["use_bcast"], b["out_len"], b["reduce_size"]) == (False, 3, 5)


# ------------------------------------------------- row slicing / format transform
def test_row_slicing_reference_vector():
    g = REF["graph_20x5"]
    v = REF["rowwise_slicing_test1"]
    ip, coo, ix, sel = O.row_slice_csc(g["indptr"], g["indices"], v["rows"])
    assert ip.tolist() == v["indptr"] and ix.tolist() == v["indices"]
    assert sel.tolist() == v["rows"] and coo.tolist() == list(range(20))


def test_row_slice_coo_closed_form():
    rng = np.random.default_rng(11)
    cases = []
    # distinct ids in random order: position != value, so value-for-position mistakes show
    key = rng.integers(0, 300, size=5000)
    cases.append((key, rng.integers(0, 10 ** 6, size=5000), rng.permutation(300)[:97]))
    # duplicate ids: first-vs-last occurrence mistakes show (3 at 0 and 2, 17 at 1 and 5)
    cases.append((key, np.arange(5000), np.array([3, 17, 3, 42, 8, 17, 299, 0])))
    # nothing kept / everything kept / ids the edges never mention / no edges / no ids
    cases.append((key, np.arange(5000), np.array([1000, 2000])))
    cases.append((key, np.arange(5000), np.arange(299, -1, -1)))
    cases.append((key, np.arange(5000), np.array([5, 100000, 7])))
    cases.append((np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64), np.array([1, 2])))
    cases.append((key, np.arange(5000), np.zeros(0, dtype=np.int64)))
    # the reference's own graph (tests/test_rowwise_slicing.cc) as a COO
    g = REF["graph_20x5"]
    indptr = np.asarray(g["indptr"])
    cases.append((np.asarray(g["indices"]), np.repeat(np.arange(indptr.size - 1), np.diff(indptr)),
                  np.asarray(REF["rowwise_slicing_test1"]["rows"])))
    for key, other, ids in cases:
        want = row_slice_coo_closed_form(key, other, ids)
        got = O.row_slice_coo(key, other, ids)
        for g_, w_ in zip(got, want):
            assert np.array_equal(g_, w_)
    # a worked example by hand: ids [7, 5, 7]; 7 -> position 2 (last), 5 -> position 1
    k, o, s = O.row_slice_coo([5, 6, 7, 5, 9, 7], [10, 11, 12, 13, 14, 15], [7, 5, 7])
    assert k.tolist() == [1, 2, 1, 2] and o.tolist() == [10, 12, 13, 15] and s.tolist() == [0, 2, 3, 5]


def test_format_transform_reference_vectors():
    g = REF["graph_12col"]
    v = REF["csc2csr_test3"]
    col = O.csc2coo(g["indptr"], 4)
    assert col.tolist() == [10, 10, 11, 11]
    ip, val, perm = O.coo2csc(g["indices"], col, 12, False)
    assert ip.tolist() == v["indptr"] and val.tolist() == v["indices"] and perm.tolist() == v["e_ids"]
    key = np.random.default_rng(1).integers(0, 50, 3000)
    value = np.arange(3000)
    ip, val, perm = O.coo2csc(key, value, 50, False)
    assert np.array_equal(perm, np.argsort(key, kind="stable")) and np.array_equal(val, value[perm])
    assert np.array_equal(ip, np.concatenate([[0], np.cumsum(np.bincount(key, minlength=50))]))


# ------------------------------------------------------- committed replay goldens
def test_oracle_reproduces_committed_goldens():
    indptr, indices, cols, probs = GOLD["indptr"], GOLD["indices"], GOLD["cols"], GOLD["probs"]
    for name, algo in (("floyd", O.ALGO_AUTO), ("reservoir", O.ALGO_RESERVOIR)):
        r = O.sample_uniform(indptr, indices, cols, 5, False, replay=GOLD[name + "_draws"],
                             with_coo=False, algo=algo)
        assert np.array_equal(r[0], GOLD[name + "_sub_indptr"])
        assert np.array_equal(r[2], GOLD[name + "_sub_indices"])
        assert np.array_equal(r[3], GOLD[name + "_select_index"])
    r = O.sample_weighted(indptr, indices, probs, cols, 4, replay=GOLD["weighted_draws"], with_coo=False)
    assert np.array_equal(r[3], GOLD["weighted_select_index"])
    tr = O.random_walk(indptr, indices, GOLD["walk_seeds"], 6, replay=GOLD["walk_draws"])
    assert np.array_equal(tr, GOLD["walk_trace"])
    fr, rel = O.relabel([cols, GOLD["floyd_sub_indices"]], [GOLD["floyd_sub_indices"]])
    assert np.array_equal(fr, GOLD["relabel_frontier"]) and np.array_equal(rel[0], GOLD["relabel_rows"])


# ------------------------------------------------- induced subgraph, super-batch
def test_col_row_slice_against_an_edge_loop():
    indptr, indices = rmat_csc_np(64, 600, seed=1)
    rng = np.random.default_rng(0)
    cols = rng.integers(0, 64, size=20)
    rows = rng.permutation(64)[:25]
    got = O.col_row_slice(indptr, indices, cols, rows)
    pos = {int(r): i for i, r in enumerate(rows)}
    ptr, idx, sel, par, p = [0], [], [], [], 0
    for c in cols:
        for e in range(indptr[c], indptr[c + 1]):
            if int(indices[e]) in pos:
                idx.append(pos[int(indices[e])])
                sel.append(p)
                par.append(e)
            p += 1
        ptr.append(len(idx))
    for g, w in zip(got, (ptr, idx, sel, par)):
        assert np.array_equal(g, w)
    # batched: rows keep their id; a column only sees the ids of its own batch
    col_ptr, row_ptr = np.array([0, 8, 20]), np.array([0, 10, 25])
    got = O.col_row_slice(indptr, indices, cols, rows, col_ptr, row_ptr, 64)
    ptr, idx = [0], []
    for r, c in enumerate(cols):
        b = 0 if r < 8 else 1
        mine = set(rows[row_ptr[b]:row_ptr[b + 1]].tolist())
        idx += [int(v) for v in indices[indptr[c]:indptr[c + 1]] if int(v) in mine]
        ptr.append(len(idx))
    assert np.array_equal(got[0], ptr) and np.array_equal(got[1], idx)


def test_batch_helpers_worked_examples():
    # two inputs, two batches: batch 0 = [1,2 | 10], batch 1 = [3,4,5 | 20,30]
    d = [np.array([1, 2, 3, 4, 5]), np.array([10, 20, 30])]
    p = [np.array([0, 2, 5]), np.array([0, 1, 3])]
    total, key, total_ptr = O.batch_concat(d, p)
    assert total.tolist() == [1, 2, 10, 3, 4, 5, 20, 30]
    assert key.tolist() == [0, 0, 0, 1, 1, 1, 1, 1] and total_ptr.tolist() == [0, 3, 8]
    back = O.batch_split(total, total_ptr, p)
    assert back[0].tolist() == [1, 2, 3, 4, 5] and back[1].tolist() == [10, 20, 30]
    # encode / decode / offsets; batch 1 is empty
    enc = O.batch_encode(np.array([5, 6, 7, 8]), np.array([0, 1, 1, 4]), 100)
    assert enc.tolist() == [5, 206, 207, 208]
    assert [a.tolist() for a in O.batch_decode(enc, 100)] == [[5, 6, 7, 8], [0, 2, 2, 2]]
    ptr, dec = O.batch_offsets(enc, 3, 100)
    assert ptr.tolist() == [0, 1, 1, 4] and dec.tolist() == [5, 6, 7, 8]
    # per-batch unique: first occurrence, or ascending
    assert [a.tolist() for a in O.batch_unique(np.array([3, 1, 3, 2, 2, 9]), np.array([0, 3, 6]))] == \
        [[3, 1, 2, 9], [0, 2, 4], [0, 0, 1, 1]]
    assert O.batch_unique(np.array([3, 1, 3, 2, 2, 9]), np.array([0, 3, 6]), sort=True)[0].tolist() == \
        [1, 3, 2, 9]
    # position lookup, last occurrence of a repeated value
    assert O.index_search(np.array([5, 6, 5]), np.array([5, 7, 6])).tolist() == [2, -1, 1]
    # COO relabel: batch 0 seeds [4], edges (7->4), (4->4); batch 1 seeds [5,6], edges (9->5), (5->6)
    u, u_ptr, row, col = O.batch_coo_relabel(np.array([4, 5, 6]), np.array([0, 1, 3]),
                                             np.array([4, 4, 5, 6]), np.array([7, 4, 9, 5]),
                                             np.array([0, 2, 4]))
    assert u.tolist() == [4, 7, 5, 6, 9] and u_ptr.tolist() == [0, 2, 5]
    assert row.tolist() == [1, 0, 2, 0] and col.tolist() == [0, 0, 0, 1]
    # batched filter: the id 3 belongs to batch 1 only
    r, c, ptr, sel = O.coo_filter(np.array([3, 4, 3, 5]), np.array([3, 4, 3, 5]), np.array([0, 1, 2, 3]),
                                  np.array([4, 3]), np.array([0, 2, 4]), np.array([0, 1, 2]))
    assert r.tolist() == [4, 3] and c.tolist() == [1, 2] and ptr.tolist() == [0, 1, 2] and sel.tolist() == [1, 2]
