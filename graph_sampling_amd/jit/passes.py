"""Rewrites of a traced sampler (a torch.fx graph of `Graph` method calls).

* `merge_relabel_and_all_indices` -- `Relabel()` and `AllValidNode()` of one graph compute the
  same frontier; one `Relabel()` serves both (python/gs/jit/optimize.py:7-59).  On a graph
  that carries a row id list (the result of a row slice) the two list the same nodes in
  different orders -- `AllValidNode` follows the id list, `Relabel` the edges
  (src/graph.cc:757-778, 782-839) -- and the merged sampler uses the block's order for the
  next layer's seeds, which is what keeps consecutive blocks aligned.
* `fuse_slicing_and_sampling` -- a column slice whose only consumer is a uniform column
  sampling becomes the fused operator that never writes the slice (optimize.py:62-82).
* `common_subexpressions` -- repeated pure queries of one graph (valid rows, sums, ...) are
  made once (python/gs/jit/passes.py:40-58, restricted here to calls known to be pure:
  sampling calls draw fresh random numbers and must stay apart).
* `dead_code` -- calls without users go, except those that change their receiver
  (python/gs/jit/passes.py:15-37).
"""
import operator

import torch.fx as fx

from ..format import _COO, _CSC

RELABEL = ("_CAPI_Relabel", "_CAPI_relabel")
ALL_VALID = ("_CAPI_AllValidNode", "_CAPI_all_valid_node")
SLICING = ("_CAPI_Slicing", "_CAPI_slicing")
SAMPLING = ("_CAPI_Sampling", "_CAPI_sampling")
FUSED = "_CAPI_FusedColumnwiseSlicingSampling"

# Graph methods that read their receiver only and return the same thing when repeated
PURE_QUERIES = frozenset(n for pair in (
    RELABEL, ALL_VALID, SLICING,
    ("_CAPI_GetRows", "_CAPI_get_rows"), ("_CAPI_GetCols", "_CAPI_get_cols"),
    ("_CAPI_GetValidRows", "_CAPI_get_valid_rows"), ("_CAPI_GetValidCols", "_CAPI_get_valid_cols"),
    ("_CAPI_GetCOORows", "_CAPI_get_coo_rows"), ("_CAPI_GetCooCols", "_CAPI_get_coo_cols"),
    ("_CAPI_GetNumRows", "_CAPI_get_num_rows"), ("_CAPI_GetNumCols", "_CAPI_get_num_cols"),
    ("_CAPI_GetNumEdges", "_CAPI_get_num_edges"), ("_CAPI_GetData", "_CAPI_get_data"),
    ("_CAPI_Sum", "_CAPI_sum"), ("_CAPI_Normalize", "_CAPI_normalize"),
    ("_CAPI_Divide", "_CAPI_divide"), ("_CAPI_GetCSC", "_CAPI_get_csc"),
    ("_CAPI_GetCOO", "_CAPI_get_coo"), ("_CAPI_GetHomoGraph", "_CAPI_get_homo_graph"),
) for n in pair)
# calls whose result differs from call to call: never merged, but removable when unused
RANDOM = frozenset((
    "_CAPI_Sampling", "_CAPI_sampling", "_CAPI_SamplingWithProbs", "_CAPI_sampling_with_probs",
    FUSED, "_CAPI_fused_columnwise_slicing_sampling", "_CAPI_RandomWalk", "_CAPI_random_walk",
    "_CAPI_MetapathRandomWalkFused", "_CAPI_metapath_random_walk_fused"))


def _is_method(node, names):
    return node.op == "call_method" and node.target in names


def _finish(gm):
    gm.graph.lint()
    gm.recompile()
    return gm


def dead_code(gm: fx.GraphModule) -> fx.GraphModule:
    """Removes value-producing calls nobody uses.  Unknown methods are kept: they may change
    their receiver (`_CAPI_SetData`, `_CAPI_SDDMM` writing into `out`, ...)."""
    for node in reversed(list(gm.graph.nodes)):
        if node.users or node.op in ("placeholder", "output"):
            continue
        removable = (node.op == "call_function" or node.op == "get_attr" or
                     _is_method(node, PURE_QUERIES) or _is_method(node, RANDOM))
        if node.op == "call_method" and not removable:
            # tensor methods (no `_CAPI_` prefix) without a trailing underscore are pure
            name = str(node.target)
            removable = not name.startswith("_CAPI_") and not name.endswith("_")
        if removable:
            gm.graph.erase_node(node)
    return _finish(gm)


def merge_relabel_and_all_indices(gm: fx.GraphModule) -> fx.GraphModule:
    groups = {}
    for node in gm.graph.nodes:
        if _is_method(node, RELABEL) or _is_method(node, ALL_VALID):
            groups.setdefault(node.args[0], []).append(node)
    for receiver, calls in groups.items():
        if len(calls) < 2 or not any(_is_method(c, RELABEL) for c in calls):
            continue
        with gm.graph.inserting_before(calls[0]):  # calls are in graph order
            relabel = gm.graph.call_method(RELABEL[0], (receiver,))
            frontier = gm.graph.call_function(operator.getitem, (relabel, 0))
        for call in calls:
            call.replace_all_uses_with(frontier if _is_method(call, ALL_VALID) else relabel)
            gm.graph.erase_node(call)
    return dead_code(gm)


def fuse_slicing_and_sampling(gm: fx.GraphModule) -> fx.GraphModule:
    for node in list(gm.graph.nodes):
        if not _is_method(node, SAMPLING) or len(node.args) != 6:
            continue
        sliced, axis, fanout, replace, on_format, _ = node.args
        if not (isinstance(sliced, fx.Node) and _is_method(sliced, SLICING) and
                len(sliced.users) == 1 and len(sliced.args) == 6):
            continue
        parent, ids, s_axis, s_on, _, s_relabel = sliced.args
        if (axis, on_format, s_axis, s_on, s_relabel) != (0, _CSC, 0, _CSC, False):
            continue
        with gm.graph.inserting_after(node):
            fused = gm.graph.call_method(FUSED, (parent, ids, fanout, replace))
        node.replace_all_uses_with(fused)
        gm.graph.erase_node(node)
        gm.graph.erase_node(sliced)
    return dead_code(gm)


def common_subexpressions(gm: fx.GraphModule) -> fx.GraphModule:
    seen = {}
    for node in list(gm.graph.nodes):
        pure = _is_method(node, PURE_QUERIES) or (
            node.op == "call_function" and node.target is operator.getitem)
        if not pure:
            continue
        key = (node.op, node.target, node.args, tuple(sorted(node.kwargs.items())))
        try:
            first = seen.setdefault(key, node)
        except TypeError:  # an unhashable argument (a list): leave the call alone
            continue
        if first is not node:
            node.replace_all_uses_with(first)
            gm.graph.erase_node(node)
    return _finish(gm)


DEFAULT = (merge_relabel_and_all_indices, fuse_slicing_and_sampling, common_subexpressions,
           dead_code)
