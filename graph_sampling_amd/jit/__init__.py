"""Trace a sampler once, rewrite it, replay it: `compile(func, args)`.

The counterpart of the reference's `gs.jit.compile` (python/gs/jit/module.py:85-137): a
sampler written against `Matrix` is traced with torch.fx into a graph of `Graph` method calls
and tensor operations, rewritten (`passes`), and replayed on every call.  Matrix arguments
enter the trace as their `Graph` handle, lists / tuples / numbers / strings (fanouts,
metapaths) are frozen into it, tensors stay arguments.

As with any torch.fx trace, the sampler's Python control flow is followed once, at compile
time: loops over the frozen arguments unroll, and a branch must not depend on the value or
the size of a tensor (such a sampler is run as it is, without `compile`).
"""
from .compiler import compile, trace  # noqa: F401
from . import passes  # noqa: F401
