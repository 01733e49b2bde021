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


def columns_as_a_graph(indptr, indices, cols, with_positions=False):
    """(offsets, neighbour ids) of the columns `cols` of a device CSC as numpy arrays, cut out
    with plain torch indexing (no library kernel).  The oracle's samplers address a column by
    its place in the call, so sampling columns 0..len(cols)-1 of this small graph with the same
    seed gives what sampling `cols` of the whole graph gives: graphs too large to copy to the
    host are checked this way.  Ids outside the graph count as empty columns.
    with_positions: also the place of every edge of the small graph in the whole graph's
    `indices` (a device tensor), which turns the oracle's select_index into the graph's."""
    import torch
    n = indptr.numel() - 1
    cols = cols.long()
    ok = (cols >= 0) & (cols < n)
    safe = torch.where(ok, cols, torch.zeros_like(cols))
    starts = indptr[safe]
    deg = torch.where(ok, indptr[safe + 1] - starts, torch.zeros_like(starts))
    offsets = torch.zeros(cols.numel() + 1, dtype=torch.int64, device=indptr.device)
    torch.cumsum(deg, 0, out=offsets[1:])
    total = int(offsets[-1])
    owner = torch.repeat_interleave(torch.arange(cols.numel(), device=indptr.device), deg,
                                    output_size=total)
    pos = torch.arange(total, device=indptr.device) - offsets[owner] + starts[owner]
    if with_positions:
        return offsets.cpu().numpy(), indices[pos].cpu().numpy().astype(np.int64), pos
    return offsets.cpu().numpy(), indices[pos].cpu().numpy().astype(np.int64)
