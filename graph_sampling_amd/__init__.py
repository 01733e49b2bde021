"""MI355X-native graph-sampling engine.

Hand-written HIP kernels behind a C ABI (``libgs_hip.so``, ``include/gs_hip.h``), a C++ host
layer that mirrors the ``gs::Graph`` / ``graph_ops`` API of czkkkkkk/graph_sampling and
registers ``torch.classes.gs_classes`` / ``torch.ops.gs_ops`` (``libgs.so``), and a thin Python
layer with the ``Matrix`` / ``HeteroMatrix`` / ``ops`` surface of the reference's ``gs`` package.

``import graph_sampling_amd as gs`` is meant to read like ``import gs``.
"""
import os

from .format import _COO, _CSC, _CSR, _DCSC, _DCSR  # noqa: F401

_PKG = os.path.dirname(os.path.abspath(__file__))
HOST_LIB = os.path.join(_PKG, "libgs.so")
_loaded = False


def load_library():
    """Registers torch.classes.gs_classes.* and torch.ops.gs_ops.* (raises if libgs.so is missing)."""
    global _loaded
    if not _loaded:
        import torch
        if not os.path.exists(HOST_LIB):
            raise RuntimeError("%s is missing: run `python -m graph_sampling_amd.build`" % HOST_LIB)
        torch.classes.load_library(HOST_LIB)
        _loaded = True


def __getattr__(name):
    # torch-dependent names are resolved lazily so that the ctypes binding
    # (graph_sampling_amd.capi) can be used without the C++ host layer
    if name in ("Graph", "HeteroGraph"):
        import torch
        load_library()
        return getattr(torch.classes.gs_classes, name)
    if name in ("Matrix", "HeteroMatrix"):
        from . import matrix_api
        return getattr(matrix_api, name)
    if name == "Block":
        from . import block
        return block.Block
    if name in ("ops", "jit"):
        import importlib
        return importlib.import_module("." + name, __name__)
    raise AttributeError(name)


def set_seed(seed):
    """Seed of the next sampling / walk call made through Graph (then seed+1, ...)."""
    import torch
    load_library()
    torch.ops.gs_ops._CAPI_SetSeed(int(seed))


def set_ordered_sums(on):
    """on: `sum(axis)` of a matrix held as a COO only sorts its edges first and adds in edge
    order, so two runs give the same bits; off (the default): it adds edge by edge with float
    atomics, faster, and a sum of three or more addends may differ in its last bit run to run."""
    import torch
    load_library()
    torch.ops.gs_ops._CAPI_SetOrderedSums(bool(on))


def _blocks_of(parts, num_layers):
    from .block import Block
    blocks = []
    per = len(parts) // num_layers  # 3, or 4 when the graph has edge data (the samples' share)
    for l in range(num_layers):
        frontier, indptr, indices = parts[per * l:per * l + 3]
        data = parts[per * l + 3] if per == 4 else None
        blocks.insert(0, Block(frontier.numel(), indptr.numel() - 1, "csc", indptr, indices, frontier,
                               weights=data))
    return parts[-per], blocks


def sample_layers(matrix, seeds, fanouts, replace=False):
    """One GraphSAGE-style minibatch in one call of the C++ layer (fused slice + sample, relabel,
    next seeds = frontier, per layer): what the per-layer loop of the reference's examples does
    (examples/graphsage/batching.py:125-138), with every layer queued on the device and the
    sizes collected once.  Returns (input_nodes, [Block, ...] innermost layer first); the draws
    are those of the loop under the same seed."""
    load_library()
    graph = getattr(matrix, "_graph", matrix)
    return _blocks_of(graph._CAPI_SampleLayers(seeds, list(fanouts), bool(replace)), len(fanouts))


def sample_blocks(matrix, seed_sets, fanouts, replace=False, workers=4, seed=0, per_call=None):
    """GraphSAGE-style minibatches sampled side by side by `workers` host threads of the C++
    layer, one stream each (fused slice + sample, relabel, next seeds = frontier, per layer).
    Returns [(input_nodes, [Block, ...] innermost layer first)] in the order of `seed_sets`;
    minibatch i draws with seeds `seed + i * len(fanouts) + layer` whichever thread runs it.
    With `per_call` the seed sets go that many at a time as super-batches (the flow of
    `sample_blocks_batched`) through one thread of the pool, which queues its next super-batch
    before it collects the one before (`workers` must be 1: super-batches side by side are
    switched off in the library); group g then draws with seeds
    `seed + g * per_call * len(fanouts) + layer`."""
    import torch
    load_library()
    graph = getattr(matrix, "_graph", matrix)
    if per_call is None:
        flat = torch.ops.gs_ops._CAPI_SampleBlocks(graph, list(seed_sets), list(fanouts),
                                                   bool(replace), int(workers), int(seed))
    else:
        flat = torch.ops.gs_ops._CAPI_SampleBlocksBatched(graph, list(seed_sets), list(fanouts),
                                                          bool(replace), int(workers),
                                                          int(per_call), int(seed))
    return [_blocks_of(parts, len(fanouts)) for parts in flat]


class _QueuedMinibatch(object):
    """A minibatch whose launches are queued; `collect()` waits for it and returns
    (input_nodes, [Block, ...]) as `sample_layers` does."""

    def __init__(self, handle, num_layers):
        self._handle, self._num_layers = handle, num_layers

    def collect(self):
        return _blocks_of(self._handle.collect(), self._num_layers)


def queue_sample_layers(matrix, seeds, fanouts, replace=False):
    """`sample_layers` in two halves: the call queues every layer's launches and returns at
    once (the draws' seeds are taken now, in call order); `.collect()` of the returned object
    waits and hands over the minibatch.  Queue minibatch i + 1 before collecting minibatch i
    and the stream never waits for the host between them.  Not in the reference."""
    load_library()
    graph = getattr(matrix, "_graph", matrix)
    fanouts = list(fanouts)
    return _QueuedMinibatch(graph._CAPI_QueueSampleLayers(seeds, fanouts, bool(replace)), len(fanouts))


class _QueuedSuperBatch(object):
    """A super-batch whose launches are queued; `collect()` waits for it and returns what
    `sample_blocks_batched` returns."""

    def __init__(self, handle, num_layers):
        self._handle, self._num_layers = handle, num_layers

    def collect(self):
        return [_blocks_of(parts, self._num_layers) for parts in self._handle.collect()]


def queue_sample_blocks_batched(matrix, seed_sets, fanouts, replace=False):
    """`sample_blocks_batched` in two halves: the call returns when the last layer's launches
    are queued, `.collect()` of the returned object waits for them and hands over the
    minibatches.  Queue super-batch i + 1 before collecting super-batch i and the host's share
    of a call (concatenating the seeds, the per-minibatch views) runs while the stream is busy.
    Not in the reference."""
    load_library()
    graph = getattr(matrix, "_graph", matrix)
    fanouts = list(fanouts)
    return _QueuedSuperBatch(
        graph._CAPI_QueueSampleLayersBatched(list(seed_sets), fanouts, bool(replace)), len(fanouts))


def sample_blocks_batched(matrix, seed_sets, fanouts, replace=False):
    """GraphSAGE-style minibatches sampled as ONE launch sequence per layer (a "super-batch": the
    flow of the reference's examples/graphsage/batching.py:59-98 -- fused sampling over the
    concatenated seeds, one relabel per minibatch done in one pass, the splits -- run inside the
    C++ layer).  Returns [(input_nodes, [Block, ...] innermost layer first)] in the order of
    `seed_sets`.  The throughput form: several times the edges per second of minibatch-by-
    minibatch calls, at the latency of the whole super-batch."""
    load_library()
    graph = getattr(matrix, "_graph", matrix)
    flat = graph._CAPI_SampleLayersBatched(list(seed_sets), list(fanouts), bool(replace))
    return [_blocks_of(parts, len(fanouts)) for parts in flat]
