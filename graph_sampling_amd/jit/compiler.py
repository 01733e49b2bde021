"""`compile`: trace, rewrite, replay (python/gs/jit/module.py:85-137, trace.py:10-32)."""
import torch
import torch.fx as fx

from ..matrix_api import HeteroMatrix, Matrix
from . import passes as _passes

_FROZEN = (list, tuple, int, float, bool, str, type(None))


def _hetero_from_handle(handle):
    return HeteroMatrix(handle)


class _Tracer(fx.Tracer):
    """A Matrix in the sampler's result is recorded as `Matrix(handle)`, so that the replay
    hands back Matrix objects where the sampler did."""

    def create_arg(self, a):
        if isinstance(a, Matrix):
            return self.create_node("call_function", Matrix, (self.create_arg(a._graph),), {})
        if isinstance(a, HeteroMatrix):
            return self.create_node("call_function", _hetero_from_handle,
                                    (self.create_arg(a._hetero_graph),), {})
        return super().create_arg(a)


def _role(arg):
    if isinstance(arg, Matrix):
        return "matrix"
    if isinstance(arg, HeteroMatrix):
        return "hetero"
    if isinstance(arg, _FROZEN):
        return "frozen"
    return "tensor"


def trace(func, args):
    """(GraphModule, roles): `func` traced with the Matrix arguments as graph handles, the
    frozen ones as constants and the rest as run-time arguments."""
    roles = [_role(a) for a in args]
    frozen = {i: a for i, a in enumerate(args) if roles[i] == "frozen"}

    def sampler(tensors, handles):
        rebuilt, t, h = [], 0, 0
        for i, role in enumerate(roles):
            if role == "frozen":
                rebuilt.append(frozen[i])
            elif role == "tensor":
                rebuilt.append(tensors[t])
                t += 1
            else:
                rebuilt.append(Matrix(handles[h]) if role == "matrix" else HeteroMatrix(handles[h]))
                h += 1
        return func(*rebuilt)

    graph = _Tracer().trace(sampler)
    return fx.GraphModule(torch.nn.Module(), graph, getattr(func, "__name__", "sampler")), roles


class compile(object):
    """`compiled = compile(sampler, example_args)`; `compiled(*args)` then replays the rewritten
    trace.  Arguments frozen at compile time (fanouts, metapaths) must be passed unchanged."""

    def __init__(self, func, args, passes=_passes.DEFAULT):
        self.gm, self._roles = trace(func, args)
        self._frozen = {i: a for i, a in enumerate(args) if self._roles[i] == "frozen"}
        for rewrite in passes:
            self.gm = rewrite(self.gm)

    def __call__(self, *args):
        if len(args) != len(self._roles):
            raise TypeError("compiled for %d arguments, got %d" % (len(self._roles), len(args)))
        tensors, handles = [], []
        for i, (role, arg) in enumerate(zip(self._roles, args)):
            if role == "frozen":
                if arg != self._frozen[i]:
                    raise ValueError("argument %d was frozen as %r at compile time, got %r"
                                     % (i, self._frozen[i], arg))
            elif role == "matrix":
                handles.append(arg._graph)
            elif role == "hetero":
                handles.append(arg._hetero_graph)
            else:
                tensors.append(arg)
        return self.gm(tensors, handles)

    @property
    def code(self):
        return self.gm.code
