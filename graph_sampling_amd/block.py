"""`Block`: the bipartite message-flow graph a sampler hands to a model, without DGL.

The reference turns the tuple of `Graph::Relabel` into a `DGLBlock`
(python/gs/matrix_api/matrix.py:40-64, python/gs/utils/to_dgl_block.py:5-27).  This container
keeps the same pieces under the same names -- `srcdata['_ID']`, `edata['_ID']`, `edata['w']`,
`num_src_nodes()`, `num_dst_nodes()`, `edges()` -- and converts between the COO and the
by-destination CSC view with the library's own format kernels.  Source nodes are the
frontier (seeds first), destination nodes its first `num_dst` entries.
"""
import torch
import torch.fx

from . import load_library


class Block(object):

    def __init__(self, num_src, num_dst, fmt, first, second, src_ids=None, e_ids=None,
                 weights=None):
        if fmt not in ("coo", "csc"):
            raise ValueError("Block format must be 'coo' or 'csc', got %r" % (fmt,))
        self._num_src, self._num_dst = int(num_src), int(num_dst)
        self._coo = (first, second, None) if fmt == "coo" else None   # (src, dst, order)
        self._csc = (first, second, None) if fmt == "csc" else None   # (indptr, src, order)
        self.srcdata, self.dstdata, self.edata = {}, {}, {}
        if src_ids is not None:
            self.srcdata["_ID"] = src_ids
            self.dstdata["_ID"] = src_ids[:self._num_dst]
        if e_ids is not None:
            self.edata["_ID"] = e_ids
        if weights is not None:
            self.edata["w"] = weights
        self.format = fmt  # the format the sampler produced; edata is in that edge order

    def num_src_nodes(self):
        return self._num_src

    def num_dst_nodes(self):
        return self._num_dst

    def num_edges(self):
        return int((self._coo[0] if self._coo is not None else self._csc[1]).numel())

    def _helper(self):
        load_library()
        g = torch.classes.gs_classes.Graph(True)
        if self._coo is not None:
            g._CAPI_LoadCOO(self._coo[0], self._coo[1])
        else:
            g._CAPI_LoadCSC(self._csc[0], self._csc[1])
        return g

    def edges(self):
        """(src, dst) local ids, in the edge order of `edata` when the block was made as COO,
        else ordered by destination (the CSC's own order, which is then `edata`'s too)."""
        if self._coo is None:
            row, col, _ = self._helper()._CAPI_GetCOO()
            self._coo = (row, col, None)
        return self._coo[0], self._coo[1]

    def csc(self):
        """(indptr over destinations, source ids, order) -- `order[i]` is the position in
        `edata` of the i-th CSC edge, or None when the orders agree."""
        if self._csc is None:
            indptr, indices, order = self._helper()._CAPI_GetCSC()
            # the helper graph sizes itself by the largest id it sees: cut or extend the
            # offsets to the block's destinations (those beyond have no edges)
            missing = self._num_dst + 1 - indptr.numel()
            if missing > 0:
                indptr = torch.cat([indptr, indptr[-1:].expand(missing)])
            elif missing < 0:
                indptr = indptr[:self._num_dst + 1]
            self._csc = (indptr, indices, order if order.numel() else None)
        return self._csc

    def in_degrees(self):
        indptr = self.csc()[0]
        return indptr[1:] - indptr[:-1]

    def adj(self, weighted=True):
        """num_dst x num_src sparse CSR matrix (edge weights, or ones), for `adj @ features`."""
        indptr, indices, order = self.csc()
        w = self.edata.get("w") if weighted else None
        if w is None:
            w = torch.ones(indices.numel(), dtype=torch.float32, device=indices.device)
        elif order is not None:
            w = w[order]
        return torch.sparse_csr_tensor(indptr, indices.long(), w,
                                       size=(self._num_dst, self._num_src))

    def __repr__(self):
        return "Block(num_src_nodes=%d, num_dst_nodes=%d, num_edges=%d, format=%s)" % (
            self._num_src, self._num_dst, self.num_edges(), self.format)


def make_block(relabel_out, data):
    """Block from the tuple of `Graph::Relabel` (src/graph.cc:782-839) and the graph's edge
    data.  Under a trace (`graph_sampling_amd.jit`) the call is recorded as one node, so what
    depends on run-time values (is there an `e_ids`? is there data?) is decided at run time."""
    if isinstance(relabel_out, torch.fx.Proxy):
        return relabel_out.tracer.create_proxy("call_function", make_block, (relabel_out, data), {})
    frontier, num_src, num_dst, first, second, e_ids, fmt = relabel_out
    if data is not None and e_ids is not None:
        data = data[e_ids]
    return Block(num_src, num_dst, fmt, first, second, frontier, e_ids, data)
