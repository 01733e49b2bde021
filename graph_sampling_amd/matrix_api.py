"""`Matrix` and `HeteroMatrix`: the Python surface of the reference's gs package
(python/gs/matrix_api/matrix.py:13-119, hetero_matrix.py:6-27), on torch.classes.gs_classes.

Method names, argument order and the format flag each method passes are those of the
reference; `to_dgl_block` returns this package's own `Block` because DGL is not a dependency.
Methods are written so that `graph_sampling_amd.jit` can trace them: no branch depends on a
tensor's value.
"""
import torch
import torch.fx

from . import block as _block
from . import load_library
from .format import _COO, _CSC, _CSR


class Matrix(object):

    def __init__(self, graph=None):
        load_library()
        self._graph = graph if graph is not None else torch.classes.gs_classes.Graph(False)

    # -- construction ------------------------------------------------------
    def load_csc(self, indptr, indices, data=None):
        self._graph._CAPI_LoadCSC(indptr, indices)
        if data is not None:
            self._graph._CAPI_SetData(data)
        return self

    def load_coo(self, row, col, data=None):
        self._graph._CAPI_LoadCOO(row, col)
        if data is not None:
            self._graph._CAPI_SetData(data)
        return self

    def set_data(self, data):
        self._graph._CAPI_SetData(data)

    def get_data(self, order='default'):
        return self._graph._CAPI_GetData(order)

    def get_num_rows(self):
        return self._graph._CAPI_GetNumRows()

    def get_num_cols(self):
        return self._graph._CAPI_GetNumCols()

    def get_num_edges(self):
        return self._graph._CAPI_GetNumEdges()

    # -- structure operators ----------------------------------------------
    def columnwise_slicing(self, t):
        return Matrix(self._graph._CAPI_Slicing(t, 0, _CSC, _COO, False))

    def columnwise_sampling(self, fanout, replace=True, bias=None):
        if bias is None:
            return Matrix(self._graph._CAPI_Sampling(0, fanout, replace, _CSC, _COO))
        return Matrix(self._graph._CAPI_SamplingWithProbs(0, bias, fanout, replace, _CSC, _COO))

    def fused_columnwise_slicing_sampling(self, seeds, fanouts, replace):
        return Matrix(self._graph._CAPI_FusedColumnwiseSlicingSampling(seeds, fanouts, replace))

    def __getitem__(self, data):
        ret = self._graph
        r_slice, c_slice = data[0], data[1]
        if isinstance(c_slice, (torch.Tensor, torch.fx.Proxy)):
            ret = ret._CAPI_Slicing(c_slice, 0, _CSC, _COO, False)
        if isinstance(r_slice, (torch.Tensor, torch.fx.Proxy)):
            ret = ret._CAPI_Slicing(r_slice, 1, _CSR, _COO, False)
        return Matrix(ret)

    def random_walk(self, seeds, walk_length):
        return self._graph._CAPI_RandomWalk(seeds, walk_length)

    # -- edge-data operators -------------------------------------------------
    def sum(self, axis, powk=1):
        return self._graph._CAPI_Sum(axis, powk, _CSC if axis == 0 else _CSR)

    def divide(self, divisor, axis):
        return Matrix(self._graph._CAPI_Divide(divisor, axis, _COO))

    def normalize(self, axis):
        return Matrix(self._graph._CAPI_Normalize(axis, _CSC if axis == 0 else _CSR))

    # -- node queries ------------------------------------------------------
    def row_ids(self, remove_isolated=True, unique=None):
        if unique is not None:  # spelling used by examples/ladies/ladies_raw.py:18
            remove_isolated = unique
        return self._graph._CAPI_GetValidRows() if remove_isolated else self._graph._CAPI_GetRows()

    def all_indices(self):
        return self._graph._CAPI_AllValidNode()

    def row_indices(self):
        return self._graph._CAPI_GetCOORows(True)

    def relabel(self):
        self._graph._CAPI_Relabel()
        return self

    def to_block(self):
        """Relabels and returns the `Block` a model consumes (the reference's `to_dgl_block`,
        python/gs/matrix_api/matrix.py:40-64, without DGL)."""
        return _block.make_block(self._graph._CAPI_Relabel(), self._graph._CAPI_GetData('default'))

    to_dgl_block = to_block


class HeteroMatrix(object):

    def __init__(self, hetero_graph=None):
        load_library()
        self._hetero_graph = (hetero_graph if hetero_graph is not None
                              else torch.classes.gs_classes.HeteroGraph())

    def load_from_homo(self, node_types, edge_types, homo_matrices):
        self._hetero_graph._CAPI_LoadFromHomo(node_types, edge_types,
                                              [m._graph for m in homo_matrices])

    def get_homo_matrix(self, etype):
        return Matrix(self._hetero_graph._CAPI_GetHomoGraph(etype))

    def metapath_random_walk(self, seeds, metapath):
        """Unfused reference path: one fused slice+sample (fanout 1, replace) per step."""
        ret = [seeds]
        for etype in metapath:
            sub = self.get_homo_matrix(etype).fused_columnwise_slicing_sampling(seeds, 1, True)
            seeds = sub.row_indices()
            ret.append(seeds)
        return torch.stack(ret)

    def metapath_random_walk_fused(self, seeds, metapath):
        return self._hetero_graph._CAPI_MetapathRandomWalkFused(seeds, metapath)
