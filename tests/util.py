"""Shared inputs for the parity tests: the reference's closed-form graphs and
seeded R-MAT graphs (numpy, CPU)."""
import numpy as np


def graph_20x5():
    """tests/test_colwise_slicing.cc:11-13 of the reference: 20 columns x 5 neighbours."""
    return np.arange(21, dtype=np.int64) * 5, np.arange(100, dtype=np.int64)


def graph_12col_4edge():
    """tests/test_graph_compute.cc:81-82 of the reference."""
    indptr = np.array([0] * 10 + [0, 2, 4], dtype=np.int64)
    indices = np.array([1, 3, 1, 3], dtype=np.int64)
    return indptr, indices


def rmat_csc_np(num_nodes, num_edges, a=0.57, b=0.19, c=0.19, seed=0):
    """Small R-MAT graph (numpy).  Returns (indptr, indices) int64, CSC by stable sort on dst."""
    rng = np.random.default_rng(seed)
    bits = max(1, int(np.ceil(np.log2(num_nodes))))
    src = np.zeros(num_edges, dtype=np.int64)
    dst = np.zeros(num_edges, dtype=np.int64)
    for _ in range(bits):
        r = rng.random(num_edges)
        sbit = r >= a + b
        dbit = ((r >= a) & (r < a + b)) | (r >= a + b + c)
        src = (src << 1) | sbit
        dst = (dst << 1) | dbit
    src %= num_nodes
    dst %= num_nodes
    perm = np.argsort(dst, kind="stable")
    indices = src[perm]
    indptr = np.zeros(num_nodes + 1, dtype=np.int64)
    np.cumsum(np.bincount(dst, minlength=num_nodes), out=indptr[1:])
    return indptr, indices


def u32_draws(n, seed):
    return np.random.default_rng(seed).integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)


def to_dev(a, dev, dtype=None):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a))
    if a.dtype == np.uint32:
        t = torch.from_numpy(np.ascontiguousarray(a).view(np.int32))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(dev)


def row_slice_coo_closed_form(key, other, ids):
    """Row slice of a COO from first principles, no oracle involved: an edge is kept when its
    key is among `ids`; the kept key is renamed to its POSITION in `ids` (the value stored by
    hashmap.Insert(key[i], i), src/cuda/slicing.cu:744; of duplicate ids the last position
    wins), the other end is carried, select_index is the edge's place in the input."""
    key, other, ids = (np.asarray(a, dtype=np.int64) for a in (key, other, ids))
    place = {int(v): i for i, v in enumerate(ids.tolist())}  # a later duplicate overwrites
    mask = np.isin(key, ids)
    renamed = np.array([place[int(v)] for v in key[mask]], dtype=np.int64)
    return renamed, other[mask], np.nonzero(mask)[0].astype(np.int64)
