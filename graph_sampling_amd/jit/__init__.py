"""Trace a sampler once, rewrite it, replay it: `compile(func, args)`.

The counterpart of the reference's `gs.jit.compile` (python/gs/jit/module.py:85-137): a
sampler written against `Matrix` is traced with torch.fx into a graph of `Graph` method calls
and tensor operations, rewritten (`passes`), and replayed on every call.  Matrix arguments
enter the trace as their `Graph` handle, lists / tuples / numbers / strings (fanouts,
metapaths) are frozen into it, tensors stay arguments.
"""
from .compiler import compile, trace  # noqa: F401
from . import passes  # noqa: F401
