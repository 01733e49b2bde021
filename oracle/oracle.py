"""ctypes front end of the CPU oracle (``gs_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, the smoke check and the
benchmark's ``cpu_baseline`` leg; never by the shipped package.

All functions take and return numpy arrays; ids are int64, edge data float32
(the reference's only instantiation, src/cuda/slicing.cu:176).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

TAG_UNIFORM, TAG_WEIGHTED, TAG_WALK, TAG_LIST_UNIFORM, TAG_LIST_WEIGHTED = 1, 2, 3, 4, 5
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "copy_lhs": 4, "copy_rhs": 5, "dot": 6}


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        args = ["make", "-C", _HERE]
        if force:
            args.append("-B")
        subprocess.check_call(args, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.gso_draw.restype = ctypes.c_uint32
        _lib.gso_draw.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_uint64]
        _lib.gso_log2_u24.restype = ctypes.c_float
        _lib.gso_log2_u24.argtypes = [ctypes.c_uint32]
        _lib.gso_ares_key.restype = ctypes.c_float
        _lib.gso_ares_key.argtypes = [ctypes.c_uint32, ctypes.c_float]
        for name in ("gso_slice_count", "gso_sample_count", "gso_weighted_replay_count",
                     "gso_list_sample_uniform", "gso_list_sample_weighted", "gso_unique",
                     "gso_relabel", "gso_row_slice_csc", "gso_row_slice_coo"):
            getattr(_lib, name).restype = ctypes.c_int64
        _lib.gso_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return int(lib().gso_num_threads())


def set_num_threads(n):
    lib().gso_set_num_threads(ctypes.c_int(int(n)))


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def _p(a):
    """pointer or NULL"""
    if a is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(a.ctypes.data)


def _c64(v):
    return ctypes.c_int64(int(v))


def _cu64(v):
    return ctypes.c_uint64(int(v) & 0xFFFFFFFFFFFFFFFF)


# ----------------------------------------------------------------------- RNG
def philox4x32_10(ctr, key):
    ctr = _u32(ctr)
    key = _u32(key)
    out = np.zeros(4, dtype=np.uint32)
    lib().gso_philox4x32_10(_p(ctr), _p(key), _p(out))
    return out


def draw(seed, tag, row, idx):
    return int(lib().gso_draw(_cu64(seed), ctypes.c_uint32(tag), _cu64(row), _cu64(idx)))


def log2_u24(x):
    return float(lib().gso_log2_u24(ctypes.c_uint32(int(x))))


def ares_key(x, w):
    return float(lib().gso_ares_key(ctypes.c_uint32(int(x)), ctypes.c_float(float(w))))


# ------------------------------------------------------------------- slicing
def slice_columns(indptr, indices, cols, with_coo=True):
    """src/cuda/slicing.cu:122-168 -> (sub_indptr, coo_col|None, sub_indices, select_index)"""
    indptr, indices, cols = _i64(indptr), _i64(indices), _i64(cols)
    S = cols.size
    sub_indptr = np.empty(S + 1, dtype=np.int64)
    nnz = lib().gso_slice_count(_p(indptr), _c64(indptr.size - 1), _p(cols), _c64(S), _p(sub_indptr))
    sub_indices = np.empty(nnz, dtype=np.int64)
    select_index = np.empty(nnz, dtype=np.int64)
    coo_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    lib().gso_slice_fill(_p(indptr), _p(indices), _p(cols), _c64(S), _p(sub_indptr),
                         _p(sub_indices), _p(select_index), _p(coo_col))
    return sub_indptr, coo_col, sub_indices, select_index


# ------------------------------------------------------------------ sampling
ALGO_AUTO, ALGO_RESERVOIR = 0, 1
FLOYD_MAX_K = 64


def sample_count(indptr, cols, k, replace, want_replay_ptr=False, algo=ALGO_AUTO):
    indptr = _i64(indptr)
    cols = None if cols is None else _i64(cols)
    S = indptr.size - 1 if cols is None else cols.size
    sub_indptr = np.empty(S + 1, dtype=np.int64)
    replay_ptr = np.empty(S + 1, dtype=np.int64) if want_replay_ptr else None
    lib().gso_sample_count(_p(indptr), _c64(indptr.size - 1), _p(cols), _c64(S), _c64(k), ctypes.c_int(int(replace)),
                           ctypes.c_int(int(algo)), _p(sub_indptr), _p(replay_ptr))
    return sub_indptr, replay_ptr


def sample_uniform(indptr, indices, cols, k, replace, seed=0, replay=None, with_coo=True,
                   algo=ALGO_AUTO):
    """src/cuda/sampling.cu:100-154 (cols=None) / fusion/slice_sampling.cu:91-143.

    algo=ALGO_RESERVOIR is the reference's Algorithm R on every row; ALGO_AUTO uses
    Floyd's selection on rows with deg > k (k <= FLOYD_MAX_K).

    Returns (sub_indptr, coo_col|None, sub_indices, select_index)."""
    indptr, indices = _i64(indptr), _i64(indices)
    cols = None if cols is None else _i64(cols)
    S = indptr.size - 1 if cols is None else cols.size
    sub_indptr, replay_ptr = sample_count(indptr, cols, k, replace,
                                          want_replay_ptr=replay is not None, algo=algo)
    nnz = int(sub_indptr[S])
    if replay is not None:
        replay = _u32(replay)
        assert replay.size >= int(replay_ptr[S])
    sub_indices = np.empty(nnz, dtype=np.int64)
    select_index = np.empty(nnz, dtype=np.int64)
    coo_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    lib().gso_sample_uniform_fill(_p(indptr), _c64(indptr.size - 1), _p(indices), _p(cols), _c64(S), _c64(k),
                                  ctypes.c_int(int(replace)), ctypes.c_int(int(algo)),
                                  _cu64(seed), _p(replay),
                                  _p(replay_ptr), _p(sub_indptr), _p(sub_indices),
                                  _p(select_index), _p(coo_col))
    return sub_indptr, coo_col, sub_indices, select_index


def sample_one_keepdim(indptr, indices, cols, seed=0, replay=None):
    """src/cuda/fusion/slice_sampling.cu:157-200 -> (sub_indptr, sub_indices, select_index)"""
    indptr, indices, cols = _i64(indptr), _i64(indices), _i64(cols)
    S = cols.size
    replay = None if replay is None else _u32(replay)
    sub_indptr = np.empty(S + 1, dtype=np.int64)
    sub_indices = np.empty(S, dtype=np.int64)
    select_index = np.empty(S, dtype=np.int64)
    lib().gso_sample_one_keepdim(_p(indptr), _c64(indptr.size - 1), _p(indices), _p(cols), _c64(S), _cu64(seed),
                                 _p(replay), _p(sub_indptr), _p(sub_indices), _p(select_index))
    return sub_indptr, sub_indices, select_index


def weighted_replay_ptr(indptr, cols, k):
    indptr = _i64(indptr)
    cols = None if cols is None else _i64(cols)
    S = indptr.size - 1 if cols is None else cols.size
    rp = np.empty(S + 1, dtype=np.int64)
    lib().gso_weighted_replay_count(_p(indptr), _c64(indptr.size - 1), _p(cols), _c64(S), _c64(k), _p(rp))
    return rp


def sample_weighted(indptr, indices, probs, cols, k, seed=0, replay=None, with_coo=True):
    """src/cuda/sampling_probs.cu:192-264 (without replacement)."""
    indptr, indices, probs = _i64(indptr), _i64(indices), _f32(probs)
    cols = None if cols is None else _i64(cols)
    S = indptr.size - 1 if cols is None else cols.size
    sub_indptr, _ = sample_count(indptr, cols, k, False)
    nnz = int(sub_indptr[S])
    replay_ptr = None
    if replay is not None:
        replay = _u32(replay)
        replay_ptr = weighted_replay_ptr(indptr, cols, k)
        assert replay.size >= int(replay_ptr[S])
    sub_indices = np.empty(nnz, dtype=np.int64)
    select_index = np.empty(nnz, dtype=np.int64)
    coo_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    lib().gso_sample_weighted_fill(_p(indptr), _c64(indptr.size - 1), _p(indices), _p(probs), _p(cols), _c64(S), _c64(k),
                                   _cu64(seed), _p(replay), _p(replay_ptr), _p(sub_indptr),
                                   _p(sub_indices), _p(select_index), _p(coo_col))
    return sub_indptr, coo_col, sub_indices, select_index


def sample_weighted_replace(indptr, indices, probs, cols, k, seed=0, replay=None, with_coo=True):
    """src/cuda/sampling_probs.cu:112-183 (with replacement, inverse CDF)."""
    indptr, indices, probs = _i64(indptr), _i64(indices), _f32(probs)
    cols = None if cols is None else _i64(cols)
    S = indptr.size - 1 if cols is None else cols.size
    sub_indptr, _ = sample_count(indptr, cols, k, True)
    nnz = int(sub_indptr[S])
    if replay is not None:
        replay = _u32(replay)
        assert replay.size >= S * k
    sub_indices = np.empty(nnz, dtype=np.int64)
    select_index = np.empty(nnz, dtype=np.int64)
    coo_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    lib().gso_sample_weighted_replace(_p(indptr), _c64(indptr.size - 1), _p(indices), _p(probs),
                                      _p(cols), _c64(S), _c64(k), _cu64(seed), _p(replay),
                                      _p(sub_indptr), _p(sub_indices), _p(select_index), _p(coo_col))
    return sub_indptr, coo_col, sub_indices, select_index


def list_sample_uniform(data, k, replace, seed=0, replay=None):
    """src/cuda/list_sampling.cu:20-77 -> (select, index)"""
    data = _i64(data)
    n = data.size
    replay = None if replay is None else _u32(replay)
    cap = max(n, k)
    out_data = np.empty(cap, dtype=np.int64)
    out_index = np.empty(cap, dtype=np.int64)
    m = lib().gso_list_sample_uniform(_p(data), _c64(n), _c64(k), ctypes.c_int(int(replace)),
                                      _cu64(seed), _p(replay), _p(out_data), _p(out_index))
    return out_data[:m].copy(), out_index[:m].copy()


def list_sample_weighted(data, probs, k, seed=0, replay=None):
    """src/cuda/list_sampling_probs.cu:11-91 (without replacement) -> (select, index)"""
    data, probs = _i64(data), _f32(probs)
    n = data.size
    replay = None if replay is None else _u32(replay)
    cap = max(n, k)
    out_data = np.empty(cap, dtype=np.int64)
    out_index = np.empty(cap, dtype=np.int64)
    m = lib().gso_list_sample_weighted(_p(data), _p(probs), _c64(n), _c64(k), _cu64(seed),
                                       _p(replay), _p(out_data), _p(out_index))
    return out_data[:m].copy(), out_index[:m].copy()


# ------------------------------------------------------------ unique/relabel
def unique(x):
    """src/cuda/unique_reindex.cu:81-151: distinct values, first-occurrence order"""
    x = _i64(x)
    out = np.empty(x.size, dtype=np.int64)
    u = lib().gso_unique(_p(x), _c64(x.size), _p(out))
    return out[:u].copy()


def relabel(mapping_tensors, to_be_relabeled):
    """src/cuda/unique_reindex.cu:179-199 -> (frontier, [relabeled...])"""
    mapping = _i64(np.concatenate([_i64(m) for m in mapping_tensors]))
    sizes = [int(np.asarray(t).size) for t in to_be_relabeled]
    query = _i64(np.concatenate([_i64(t) for t in to_be_relabeled])) if sizes else np.empty(0, np.int64)
    frontier = np.empty(mapping.size, dtype=np.int64)
    out = np.empty(query.size, dtype=np.int64)
    u = lib().gso_relabel(_p(mapping), _c64(mapping.size), _p(query), _c64(query.size),
                          _p(frontier), _p(out))
    outs, off = [], 0
    for s in sizes:
        outs.append(out[off:off + s].copy())
        off += s
    return frontier[:u].copy(), outs


# --------------------------------------------------------------------- walks
def batch_csr_relabel(seeds, seeds_ptr, indices, indices_ptr):
    """src/cuda/batch_relabel.cu:236-328: one relabel per batch, results concatenated.

    Returns (unique, unique_ptr, relabelled indices): batch b's frontier is the distinct values
    of (its seeds, then its indices) in first-occurrence order, and its indices are renamed to
    their rank inside that frontier."""
    seeds, indices = _i64(seeds), _i64(indices)
    seeds_ptr, indices_ptr = _i64(seeds_ptr), _i64(indices_ptr)
    uniques, outs, ptr = [], [], [0]
    for b in range(seeds_ptr.size - 1):
        s_b = seeds[seeds_ptr[b]:seeds_ptr[b + 1]]
        i_b = indices[indices_ptr[b]:indices_ptr[b + 1]]
        frontier, (rel,) = relabel([s_b, i_b], [i_b])
        uniques.append(frontier)
        outs.append(rel)
        ptr.append(ptr[-1] + frontier.size)
    cat = lambda xs: np.concatenate(xs) if xs else np.empty(0, np.int64)  # noqa: E731
    return cat(uniques), np.asarray(ptr, dtype=np.int64), cat(outs)


def batch_coo_relabel(seeds, seeds_ptr, coo_col, coo_row, coo_ptr):
    """src/cuda/batch_relabel.cu:377-480: per batch, frontier = distinct (seeds, then coo_row)
    in first-occurrence order; rows and columns renamed to their rank in it (-1 when absent).

    Returns (unique, unique_ptr, out_row, out_col)."""
    seeds, coo_col, coo_row = _i64(seeds), _i64(coo_col), _i64(coo_row)
    seeds_ptr, coo_ptr = _i64(seeds_ptr), _i64(coo_ptr)
    uniques, rows, cols, ptr = [], [], [], [0]
    for b in range(seeds_ptr.size - 1):
        s_b = seeds[seeds_ptr[b]:seeds_ptr[b + 1]]
        r_b = coo_row[coo_ptr[b]:coo_ptr[b + 1]]
        c_b = coo_col[coo_ptr[b]:coo_ptr[b + 1]]
        frontier, (rel_r, rel_c) = relabel([s_b, r_b], [r_b, c_b])
        uniques.append(frontier)
        rows.append(rel_r)
        cols.append(rel_c)
        ptr.append(ptr[-1] + frontier.size)
    cat = lambda xs: np.concatenate(xs) if xs else np.empty(0, np.int64)  # noqa: E731
    return cat(uniques), np.asarray(ptr, dtype=np.int64), cat(rows), cat(cols)


# -------------------------------------------------------- super-batch helpers
def _batch_ids(ptr, n):
    ptr = _i64(ptr)
    return np.repeat(np.arange(ptr.size - 1, dtype=np.int64), np.diff(ptr))[:n]


def batch_encode(data, ptr, encoding_size):
    """src/cuda/batch_coding.cu:11-28,74-94: data[i] + batch(i) * encoding_size"""
    data = _i64(data)
    return data + _batch_ids(ptr, data.size) * encoding_size


def batch_decode(data, encoding_size):
    """src/cuda/batch_coding.cu:96-108 -> (in mod size, in // size)"""
    data = _i64(data)
    batch = data // encoding_size
    return data - batch * encoding_size, batch


def batch_offsets(data, num_batches, encoding_size):
    """src/cuda/batch_coding.cu:110-120 -> (ptr, decoded): ptr[b+1] = #items of batch <= b"""
    decoded, batch = batch_decode(data, encoding_size)
    ptr = np.zeros(num_batches + 1, dtype=np.int64)
    ptr[1:] = np.searchsorted(batch, np.arange(num_batches), side="right")
    return ptr, decoded


def batch_concat(datas, ptrs):
    """src/cuda/batch_concat.cu:13-119 -> (total, key, total_ptr): batch b of the result is
    batch b of every input, one input after the other"""
    datas, ptrs = [_i64(d) for d in datas], [_i64(p) for p in ptrs]
    nb = ptrs[0].size - 1
    total, key = [], []
    for b in range(nb):
        for d, p in zip(datas, ptrs):
            total.append(d[p[b]:p[b + 1]])
            key.append(np.full(p[b + 1] - p[b], b, dtype=np.int64))
    cat = lambda xs: np.concatenate(xs) if xs else np.empty(0, np.int64)  # noqa: E731
    return cat(total), cat(key), np.sum(ptrs, axis=0).astype(np.int64)


def batch_split(data, data_ptr, out_ptrs):
    """src/cuda/batch_split2.cu:12-100: the inverse of batch_concat -> list of segments"""
    data, data_ptr = _i64(data), _i64(data_ptr)
    out_ptrs = [_i64(p) for p in out_ptrs]
    outs = [np.empty(p[-1], dtype=np.int64) for p in out_ptrs]
    for b in range(data_ptr.size - 1):
        at = data_ptr[b]
        for o, p in zip(outs, out_ptrs):
            n = p[b + 1] - p[b]
            o[p[b]:p[b + 1]] = data[at:at + n]
            at += n
    return outs


def batch_unique(data, data_ptr, sort=False):
    """src/cuda/batch_unique.cu:131-207 (first-occurrence order) and, with sort, what
    :209-275 is for (ascending inside every batch) -> (unique, unique_ptr, unique_key)"""
    data, data_ptr = _i64(data), _i64(data_ptr)
    uniques, ptr = [], [0]
    for b in range(data_ptr.size - 1):
        u = unique(data[data_ptr[b]:data_ptr[b + 1]])
        uniques.append(np.sort(u) if sort else u)
        ptr.append(ptr[-1] + u.size)
    out = np.concatenate(uniques) if uniques else np.empty(0, np.int64)
    ptr = np.asarray(ptr, dtype=np.int64)
    return out, ptr, _batch_ids(ptr, out.size)


def coo_filter(key, row, col, ids, key_ptr=None, ids_ptr=None):
    """src/cuda/batch_slicing.cu:150-232 (batched) and :281-329 (one id set): the edges
    whose key is among the ids (of their own batch), ids kept
    -> (row, col, offsets of the batches | None, select_index)"""
    key, row, col, ids = _i64(key), _i64(row), _i64(col), _i64(ids)
    if key_ptr is None:
        keep = np.isin(key, ids)
        out_ptr = None
    else:
        key_ptr, ids_ptr = _i64(key_ptr), _i64(ids_ptr)
        keep = np.zeros(key.size, dtype=bool)
        for b in range(key_ptr.size - 1):
            lo, hi = key_ptr[b], key_ptr[b + 1]
            keep[lo:hi] = np.isin(key[lo:hi], ids[ids_ptr[b]:ids_ptr[b + 1]])
        out_ptr = np.concatenate([[0], np.cumsum(keep)])[key_ptr].astype(np.int64)
    sel = np.flatnonzero(keep).astype(np.int64)
    return row[sel], col[sel], out_ptr, sel


def index_search(data, keys):
    """src/cuda/index_search.cu:83-140, src/tensor_ops.cc:24-33: position of every key in
    data, -1 when absent (the last position of a repeated value)"""
    uniq, last = _last_position_lookup(_i64(data))
    return _lookup(uniq, last, _i64(keys))


def random_walk(indptr, indices, seeds, length, seed=0, replay=None):
    """src/cuda/fusion/random_walk.cu:52-68 -> flat trace, memory [L+1][n]"""
    indptr, indices, seeds = _i64(indptr), _i64(indices), _i64(seeds)
    n = seeds.size
    replay = None if replay is None else _u32(replay)
    trace = np.empty((length + 1) * n, dtype=np.int64)
    lib().gso_random_walk(_p(indptr), _c64(indptr.size - 1), _p(indices), _p(seeds), _c64(n), _c64(length),
                          _cu64(seed), _p(replay), _p(trace))
    return trace


def metapath_walk(indptrs, indicess, metapath, seeds, seed=0, replay=None):
    """src/cuda/fusion/metapath_random_walk.cu:49-67 -> flat trace [L+1][n]"""
    indptrs = [_i64(a) for a in indptrs]
    indicess = [_i64(a) for a in indicess]
    metapath, seeds = _i64(metapath), _i64(seeds)
    n, L = seeds.size, metapath.size
    replay = None if replay is None else _u32(replay)
    PtrArr = ctypes.c_void_p * len(indptrs)
    ip = PtrArr(*[a.ctypes.data for a in indptrs])
    ix = PtrArr(*[a.ctypes.data for a in indicess])
    trace = np.empty((L + 1) * n, dtype=np.int64)
    nn = np.array([a.size - 1 for a in indptrs], dtype=np.int64)
    lib().gso_metapath_walk(ip, ix, _p(nn), _p(metapath), _c64(L), _p(seeds), _c64(n), _cu64(seed),
                            _p(replay), _p(trace))
    return trace


# --------------------------------------------------------------------- SDDMM
def calc_bcast(op, lhs_shape, rhs_shape):
    """Broadcast offsets; restates src/bcast.cc:10-75.

    Returns dict(use_bcast, lhs_len, rhs_len, out_len, reduce_size, lhs_off, rhs_off)."""
    lhs_len = int(np.prod(lhs_shape[1:], dtype=np.int64)) if len(lhs_shape) > 1 else 1
    rhs_len = int(np.prod(rhs_shape[1:], dtype=np.int64)) if len(rhs_shape) > 1 else 1
    use = False
    if op not in ("copy_lhs", "copy_rhs"):
        if len(lhs_shape) != len(rhs_shape):
            use = True
        else:
            use = any(lhs_shape[i] != rhs_shape[i] for i in range(1, len(lhs_shape)))
    reduce_size = 1
    lhs_off = rhs_off = None
    if use:
        max_ndim = max(len(lhs_shape), len(rhs_shape)) - 1
        out_len, j = 1, 0
        if op == "dot":
            reduce_size = lhs_shape[-1]
            j = 1
        stride_l = stride_r = 1
        lo, ro = [0], [0]
        while j < max_ndim:
            dl = 1 if len(lhs_shape) - 1 - j < 1 else lhs_shape[len(lhs_shape) - 1 - j]
            dr = 1 if len(rhs_shape) - 1 - j < 1 else rhs_shape[len(rhs_shape) - 1 - j]
            for i in range(1, max(dl, dr)):
                for k in range(out_len):
                    lo.append(lo[k] + i * (1 if i < dl else 0) * stride_l)
                    ro.append(ro[k] + i * (1 if i < dr else 0) * stride_r)
            out_len *= max(dl, dr)
            stride_l *= dl
            stride_r *= dr
            j += 1
        lhs_off, rhs_off = np.array(lo, dtype=np.int64), np.array(ro, dtype=np.int64)
    else:
        out_len = rhs_len if op == "copy_rhs" else lhs_len
        if op == "dot":
            reduce_size = lhs_shape[-1]
            out_len //= reduce_size
    return dict(use_bcast=use, lhs_len=lhs_len, rhs_len=rhs_len, out_len=out_len,
                reduce_size=reduce_size, lhs_off=lhs_off, rhs_off=rhs_off)


def sddmm_coo(op, row, col, e_ids, lhs, rhs, lhs_target, rhs_target, out=None):
    """src/cuda/sddmm.cu:280-291; lhs/rhs are [n, ...] float32 arrays"""
    row, col = _i64(row), _i64(col)
    e_ids = None if e_ids is None else _i64(e_ids)
    lhs, rhs = _f32(lhs), _f32(rhs)
    lhs2 = lhs.reshape(lhs.shape[0], -1) if lhs.ndim > 1 else lhs.reshape(-1, 1)
    rhs2 = rhs.reshape(rhs.shape[0], -1) if rhs.ndim > 1 else rhs.reshape(-1, 1)
    ls = lhs.shape if lhs.ndim > 1 else lhs.shape + (1,)
    rs = rhs.shape if rhs.ndim > 1 else rhs.shape + (1,)
    b = calc_bcast(op, ls, rs)
    E = row.size
    if out is None:
        out = np.zeros((E, b["out_len"]), dtype=np.float32)
    lib().gso_sddmm_coo(ctypes.c_int(OPS[op]), _p(row), _p(col), _p(e_ids), _c64(E), _p(lhs2),
                        _p(rhs2), _p(out), ctypes.c_int(lhs_target), ctypes.c_int(rhs_target),
                        _c64(b["lhs_len"]), _c64(b["rhs_len"]), _c64(b["out_len"]),
                        _c64(b["reduce_size"]), _p(b["lhs_off"]), _p(b["rhs_off"]))
    return out


def sddmm_csc(op, indptr, indices, e_ids, nid_map, lhs, rhs, lhs_target, rhs_target, out=None):
    """src/cuda/sddmm.cu:263-278"""
    indptr, indices = _i64(indptr), _i64(indices)
    e_ids = None if e_ids is None else _i64(e_ids)
    nid_map = None if nid_map is None else _i64(nid_map)
    lhs, rhs = _f32(lhs), _f32(rhs)
    lhs2 = lhs.reshape(lhs.shape[0], -1) if lhs.ndim > 1 else lhs.reshape(-1, 1)
    rhs2 = rhs.reshape(rhs.shape[0], -1) if rhs.ndim > 1 else rhs.reshape(-1, 1)
    ls = lhs.shape if lhs.ndim > 1 else lhs.shape + (1,)
    rs = rhs.shape if rhs.ndim > 1 else rhs.shape + (1,)
    b = calc_bcast(op, ls, rs)
    E = indices.size
    if out is None:
        out = np.zeros((E, b["out_len"]), dtype=np.float32)
    lib().gso_sddmm_csc(ctypes.c_int(OPS[op]), _p(indptr), _p(indices), _p(e_ids), _p(nid_map),
                        _c64(indptr.size - 1), _p(lhs2), _p(rhs2), _p(out),
                        ctypes.c_int(lhs_target), ctypes.c_int(rhs_target), _c64(b["lhs_len"]),
                        _c64(b["rhs_len"]), _c64(b["out_len"]), _c64(b["reduce_size"]),
                        _p(b["lhs_off"]), _p(b["rhs_off"]))
    return out


# --------------------------------------------------------------- segment ops
def segment_sum(indptr, e_ids, n_ids, data, powk, out_size):
    """src/cuda/graph_ops.cu:66-98"""
    indptr, data = _i64(indptr), _f32(data)
    e_ids = None if e_ids is None else _i64(e_ids)
    n_ids = None if n_ids is None else _i64(n_ids)
    out = np.zeros(out_size, dtype=np.float32)
    lib().gso_segment_sum(_p(indptr), _p(e_ids), _p(n_ids), _p(data), _c64(indptr.size - 1),
                          _c64(powk), _p(out))
    return out


def coo_sum(target, e_ids, data, powk, out_size):
    """src/cuda/graph_ops.cu:100-125"""
    target, data = _i64(target), _f32(data)
    e_ids = None if e_ids is None else _i64(e_ids)
    out = np.zeros(out_size, dtype=np.float32)
    lib().gso_coo_sum(_p(target), _p(e_ids), _p(data), _c64(target.size), _c64(powk), _p(out))
    return out


def segment_normalize(indptr, e_ids, data):
    """src/cuda/graph_ops.cu:160-188"""
    indptr, data = _i64(indptr), _f32(data)
    e_ids = None if e_ids is None else _i64(e_ids)
    out = np.empty_like(data)
    lib().gso_segment_normalize(_p(indptr), _p(e_ids), _p(data), _c64(indptr.size - 1), _p(out))
    return out


def e_div_u_sum(row, col, data, divisor, num_cols):
    """src/cuda/fusion/edge_map_reduce.cu:10-25 -> (out_data, out_sum)"""
    row, col, data, divisor = _i64(row), _i64(col), _f32(data), _f32(divisor)
    out_data = np.zeros(row.size, dtype=np.float32)
    out_sum = np.zeros(num_cols, dtype=np.float32)
    lib().gso_e_div_u_sum(_p(row), _p(col), _p(data), _p(divisor), _c64(row.size), _p(out_data),
                          _p(out_sum))
    return out_data, out_sum


# --------------------------------------------------------------- row slicing
def row_slice_csc(indptr, indices, row_ids, with_coo=True):
    """src/cuda/slicing.cu:463-539 -> (out_indptr, coo_col|None, out_indices, select_index)"""
    indptr, indices, row_ids = _i64(indptr), _i64(indices), _i64(row_ids)
    n = indptr.size - 1
    out_indptr = np.empty(n + 1, dtype=np.int64)
    out_indices = np.empty(indices.size, dtype=np.int64)
    select_index = np.empty(indices.size, dtype=np.int64)
    coo_col = np.empty(indices.size, dtype=np.int64) if with_coo else None
    m = lib().gso_row_slice_csc(_p(indptr), _p(indices), _c64(n), _p(row_ids), _c64(row_ids.size),
                                _p(out_indptr), _p(out_indices), _p(select_index), _p(coo_col))
    return (out_indptr, None if coo_col is None else coo_col[:m].copy(), out_indices[:m].copy(),
            select_index[:m].copy())


def row_slice_coo(key, other, ids):
    """src/cuda/slicing.cu:727-766 -> (relabeled key, other, select_index)"""
    key, other, ids = _i64(key), _i64(other), _i64(ids)
    ok = np.empty(key.size, dtype=np.int64)
    oo = np.empty(key.size, dtype=np.int64)
    sel = np.empty(key.size, dtype=np.int64)
    m = lib().gso_row_slice_coo(_p(key), _p(other), _c64(key.size), _p(ids), _c64(ids.size),
                                _p(ok), _p(oo), _p(sel))
    return ok[:m].copy(), oo[:m].copy(), sel[:m].copy()


def _last_position_lookup(ids):
    """(sorted distinct ids, position of the LAST occurrence of each)"""
    n = ids.size
    uniq, first_rev = np.unique(ids[::-1], return_index=True)
    return uniq, (n - 1 - first_rev).astype(np.int64)


def _lookup(uniq, vals, x):
    """vals[i] where uniq[i] == x, else -1"""
    if uniq.size == 0:
        return np.full(x.shape, -1, dtype=np.int64)
    pos = np.minimum(np.searchsorted(uniq, x), uniq.size - 1)
    return np.where(uniq[pos] == x, vals[pos], -1).astype(np.int64)


def col_row_slice(indptr, indices, cols, row_ids, col_ptr=None, row_ptr=None, encoding_size=0):
    """src/cuda/fusion/column_row_slicing.cu:147-211 (one id set: kept rows renamed to their
    position in row_ids) and :277-355 (batched: key id + b*encoding_size, rows keep their id)
    -> (out_indptr, out_indices, select_index, parent_index).

    select_index is what the reference returns, nonzero(out_mask): positions in the virtual
    column slice (:204-209).  parent_index is the position of the same edge in `indices`."""
    indptr, indices, cols, row_ids = _i64(indptr), _i64(indices), _i64(cols), _i64(row_ids)
    sub_indptr, coo_col, sub_indices, parent = slice_columns(indptr, indices, cols, with_coo=True)
    if col_ptr is None:
        uniq, last = _last_position_lookup(row_ids)
        val = _lookup(uniq, last, sub_indices)
    else:
        col_ptr, row_ptr = _i64(col_ptr), _i64(row_ptr)
        nb = col_ptr.size - 1
        row_batch = np.repeat(np.arange(nb, dtype=np.int64), np.diff(row_ptr))
        col_batch = np.repeat(np.arange(nb, dtype=np.int64), np.diff(col_ptr))
        uniq = np.unique(row_ids + row_batch * encoding_size)
        found = _lookup(uniq, np.zeros(uniq.size, np.int64),
                        sub_indices + col_batch[coo_col] * encoding_size)
        val = np.where(found == 0, sub_indices, -1)
    keep = val >= 0
    select_index = np.flatnonzero(keep).astype(np.int64)
    kept_before = np.concatenate([[0], np.cumsum(keep)]).astype(np.int64)
    return kept_before[sub_indptr], val[keep], select_index, parent[select_index]


# ---------------------------------------------------------- format transform
def csc2coo(indptr, nnz):
    """src/cuda/format_transform.cu:35-46 -> col vector"""
    indptr = _i64(indptr)
    col = np.empty(nnz, dtype=np.int64)
    lib().gso_csc2coo(_p(indptr), _c64(indptr.size - 1), _p(col))
    return col


def coo2csc(key, value, num_keys, is_sorted):
    """src/cuda/format_transform.cu:135-156 -> (indptr, sorted value, perm|None)"""
    key, value = _i64(key), _i64(value)
    indptr = np.empty(num_keys + 1, dtype=np.int64)
    out_value = np.empty(key.size, dtype=np.int64)
    perm = None if is_sorted else np.empty(key.size, dtype=np.int64)
    lib().gso_coo2csc(_p(key), _p(value), _c64(key.size), _c64(num_keys),
                      ctypes.c_int(int(is_sorted)), _p(indptr), _p(out_value), _p(perm))
    return indptr, out_value, perm
