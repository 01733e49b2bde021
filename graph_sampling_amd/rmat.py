"""Synthetic R-MAT graphs in CSC form (benchmark and test input; torch ops only).

R-MAT (Chakrabarti et al., SDM'04): every edge picks one quadrant per id bit,
a = (src 0, dst 0), b = (0, 1), c = (1, 0), d = (1, 1).  Ids are folded modulo
``num_nodes`` when it is not a power of two; multi-edges and self loops stay.
The CSC is built by a stable sort on the destination, so the neighbours of a
column keep generation order.
"""
import math

import torch


def rmat_edges(num_nodes, num_edges, a=0.57, b=0.19, c=0.19, seed=0, device="cpu",
               num_src_nodes=None, chunk=1 << 26):
    """Returns (src, dst) int64 tensors of length num_edges on `device`.

    num_src_nodes: size of the source side for a bipartite relation (default: num_nodes)."""
    n_dst = int(num_nodes)
    n_src = int(num_src_nodes) if num_src_nodes is not None else n_dst
    bits = max(1, int(math.ceil(math.log2(max(n_src, n_dst)))))
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    src = torch.empty(num_edges, dtype=torch.int64, device=device)
    dst = torch.empty(num_edges, dtype=torch.int64, device=device)
    for lo in range(0, num_edges, chunk):
        hi = min(num_edges, lo + chunk)
        s = torch.zeros(hi - lo, dtype=torch.int64, device=device)
        d = torch.zeros(hi - lo, dtype=torch.int64, device=device)
        for _ in range(bits):
            r = torch.rand(hi - lo, generator=gen, device=device)
            sbit = r >= (a + b)
            dbit = ((r >= a) & (r < a + b)) | (r >= a + b + c)
            s = (s << 1) | sbit.to(torch.int64)
            d = (d << 1) | dbit.to(torch.int64)
        src[lo:hi] = s % n_src
        dst[lo:hi] = d % n_dst
    return src, dst


def edges_to_csc(src, dst, num_cols, index_dtype=torch.int64):
    """(indptr int64 [num_cols+1], indices index_dtype [E]) by stable sort on dst."""
    dst_sorted, perm = torch.sort(dst, stable=True)
    indices = src[perm].to(index_dtype)
    counts = torch.bincount(dst_sorted, minlength=num_cols)
    indptr = torch.zeros(num_cols + 1, dtype=torch.int64, device=dst.device)
    torch.cumsum(counts, 0, out=indptr[1:])
    return indptr, indices


def rmat_csc(num_nodes, num_edges, a=0.57, b=0.19, c=0.19, seed=0, device="cpu",
             index_dtype=torch.int64, num_src_nodes=None):
    src, dst = rmat_edges(num_nodes, num_edges, a, b, c, seed, device, num_src_nodes)
    return edges_to_csc(src, dst, num_nodes, index_dtype)
