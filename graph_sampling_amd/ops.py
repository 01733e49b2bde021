"""Generalised SDDMM front end: gsddmm and the generated u_add_v ... e_dot_v helpers
(surface of the reference's python/gs/ops/sddmm.py:35-131 and sparse.py:14-129)."""
import sys
from itertools import product

import torch

from .format import _COO

__all__ = ['gsddmm']

_TARGET = {'u': 0, 'e': 1, 'v': 2, 'src': 0, 'edge': 1, 'dst': 2}


def infer_broadcast_shape(op, shp1, shp2):
    """Feature shape of the result (NumPy broadcasting; dot folds the last axis to 1)."""
    if op == "dot" and shp1[-1] != shp2[-1]:
        raise ValueError("Dot operator is only available for arrays with the same size on last "
                         "dimension, but got {} and {}.".format(shp1, shp2))
    n = max(len(shp1), len(shp2))
    p1 = (1,) * (n - len(shp1)) + tuple(shp1)
    p2 = (1,) * (n - len(shp2)) + tuple(shp2)
    for d1, d2 in zip(p1, p2):
        if d1 != d2 and d1 != 1 and d2 != 1:
            raise ValueError("Feature shapes {} and {} are not valid for broadcasting.".format(shp1, shp2))
    out = tuple(max(d1, d2) for d1, d2 in zip(p1, p2))
    return out[:-1] + (1,) if op == "dot" else out


def _pad_dims(lhs, rhs):
    """(N, 3, 1) with (E, 5, 3, 4) -> (N, 1, 3, 1): same number of feature axes."""
    if lhs.dim() != rhs.dim():
        n = max(lhs.dim(), rhs.dim())
        lhs = lhs.view((lhs.shape[0],) + (1,) * (n - lhs.dim()) + tuple(lhs.shape[1:]))
        rhs = rhs.view((rhs.shape[0],) + (1,) * (n - rhs.dim()) + tuple(rhs.shape[1:]))
    return lhs, rhs


def gsddmm(g, op, lhs_data, rhs_data, lhs_target='u', rhs_target='v', on_format=_COO):
    """x_e = op(x_lhs, x_rhs) for every edge of the Matrix `g`; returns the edge feature.

    sub is computed as add(-rhs) and div as mul(1/rhs), as the reference does
    (python/gs/ops/sparse.py:123-128)."""
    if lhs_data.device != rhs_data.device:
        raise ValueError("The operands data device don't match: {} and {}".format(
            lhs_data.device, rhs_data.device))
    if lhs_data.dtype != rhs_data.dtype:
        raise ValueError("The operands data type don't match: {} and {}".format(
            lhs_data.dtype, rhs_data.dtype))
    lhs, rhs = _pad_dims(lhs_data, rhs_data)
    if op == 'sub':
        op, rhs = 'add', -rhs
    elif op == 'div':
        op, rhs = 'mul', 1. / rhs
    squeeze = lhs.dim() == 1 and rhs.dim() == 1
    if lhs.dim() == 1:
        lhs = lhs.unsqueeze(-1)
    if rhs.dim() == 1:
        rhs = rhs.unsqueeze(-1)
    gidx = g._graph
    num_edges = gidx._CAPI_GetNumEdges()
    out = torch.zeros((num_edges,) + infer_broadcast_shape(op, lhs.shape[1:], rhs.shape[1:]),
                      dtype=lhs.dtype, device=lhs.device)
    if num_edges > 0:
        gidx._CAPI_SDDMM(op, lhs.contiguous(), rhs.contiguous(), out, _TARGET[lhs_target],
                         _TARGET[rhs_target], on_format)
    return out.squeeze(-1) if squeeze else out


def _make(lhs_target, rhs_target, binary_op):
    def func(g, x, y, on_format=_COO):
        return gsddmm(g, binary_op, x, y, lhs_target=lhs_target, rhs_target=rhs_target,
                      on_format=on_format)
    func.__name__ = "{}_{}_{}".format(lhs_target, binary_op, rhs_target)
    func.__doc__ = "Edge feature = {} of the {} and {} features.".format(binary_op, lhs_target, rhs_target)
    return func


for _l, _r in product("uve", "uve"):
    if _l != _r:
        for _op in ("add", "sub", "mul", "div", "dot"):
            _f = _make(_l, _r, _op)
            setattr(sys.modules[__name__], _f.__name__, _f)
            __all__.append(_f.__name__)
