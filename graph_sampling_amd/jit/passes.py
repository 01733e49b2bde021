"""Rewrites of a traced sampler (a torch.fx graph of `Graph` method calls).

* `merge_relabel_and_all_indices` -- `Relabel()` and `AllValidNode()` of one graph compute the
  same frontier; one `Relabel()` serves both (python/gs/jit/optimize.py:7-59).  On a graph
  that carries a row id list (the result of a row slice) the two list the same nodes in
  different orders -- `AllValidNode` follows the id list, `Relabel` the edges
  (src/graph.cc:757-778, 782-839) -- and the merged sampler uses the block's order for the
  next layer's seeds, which is what keeps consecutive blocks aligned.
* `fuse_slicing_and_sampling` -- a column slice whose only consumer is a uniform column
  sampling becomes the fused operator that never writes the slice (optimize.py:62-82).
* `chain_sampled_layers` -- consecutive layers of the GraphSAGE loop (fused slice + sample of
  one graph, `Relabel`, next seeds = the frontier; examples/graphsage/batching.py:125-138)
  become one `sample_layer_chain` call, which queues every layer on the device at once where
  the graph allows it and goes layer by layer where it does not.  Not in the reference.
* `fuse_layerwise_block` -- a whole layer of a layer-wise sampler (column slice, row
  probabilities, weighted pick of rows, node set, row slice, division by the probabilities,
  column normalisation, block: examples/ladies/ladies_raw.py:10-25) whose intermediate
  results serve nothing else becomes one `layerwise_block` call, which hands the layer to one
  call of the C++ layer where the graph allows it and runs the same chain where it does not.
  Not in the reference.
* `common_subexpressions` -- repeated pure queries of one graph (valid rows, sums, ...) are
  made once (python/gs/jit/passes.py:40-58, restricted here to calls known to be pure:
  sampling calls draw fresh random numbers and must stay apart).
* `dead_code` -- calls without users go, except those that change their receiver
  (python/gs/jit/passes.py:15-37).
"""
import operator

import torch
import torch.fx as fx

from ..format import _COO, _CSC, _CSR

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


def sample_layer_chain(graph, seeds, fanouts, replace):
    """[(tuple of `Graph::Relabel`, edge data)] per layer of a GraphSAGE-style minibatch, the
    values the per-layer calls `_CAPI_FusedColumnwiseSlicingSampling` -> `_CAPI_Relabel` /
    `_CAPI_GetData('default')` give under the same seed.  A root graph takes the whole
    minibatch in one call of the C++ layer; its blocks have no edge ids, and as edge data the
    sampled edges' share of the graph's, or ones on a graph without data, as the per-layer
    calls find there (src/graph.cc:68-73)."""
    fanouts = list(fanouts)
    parts = graph._CAPI_SampleLayersIfQueued(seeds, fanouts, bool(replace))
    layers = []
    if parts:
        num_dst = seeds.numel()
        per = len(parts) // len(fanouts)  # 4 with edge data
        for l in range(len(fanouts)):
            frontier, indptr, indices = parts[per * l:per * l + 3]
            data = parts[per * l + 3] if per == 4 else torch.ones(
                indices.numel(), dtype=torch.float32, device=indices.device)
            layers.append(((frontier, frontier.numel(), num_dst, indptr, indices, None, "csc"), data))
            num_dst = frontier.numel()
        return layers
    for k in fanouts:
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(seeds, k, replace)
        relabel = sub._CAPI_Relabel()
        layers.append((relabel, sub._CAPI_GetData("default")))
        seeds = relabel[0]
    return layers


def _layer_of(fused):
    """(relabel, [data queries]) when `fused` is used for its block only, else None."""
    relabel, data = None, []
    for user in fused.users:
        if _is_method(user, RELABEL) and relabel is None and user.args == (fused,):
            relabel = user
        elif (_is_method(user, ("_CAPI_GetData", "_CAPI_get_data")) and
              user.args == (fused, "default") and not user.kwargs):
            data.append(user)
        else:
            return None
    return (relabel, data) if relabel is not None else None


def chain_sampled_layers(gm: fx.GraphModule) -> fx.GraphModule:
    layer_of = {n: _layer_of(n) for n in gm.graph.nodes
                if _is_method(n, (FUSED,)) and len(n.args) == 4 and not n.kwargs}
    layer_of = {n: l for n, l in layer_of.items() if l is not None}

    def follower(fused):
        # the layer whose seeds are this layer's frontier, on the same graph and replace flag
        for item in layer_of[fused][0].users:
            if not (item.op == "call_function" and item.target is operator.getitem and
                    item.args[1] == 0):
                continue
            for nxt in item.users:
                if (nxt in layer_of and nxt.args[1] is item and nxt.args[0] is fused.args[0] and
                        nxt.args[3] == fused.args[3] and isinstance(nxt.args[2], int)):
                    return nxt
        return None

    followers = {n: follower(n) for n in layer_of}
    followed = set(f for f in followers.values() if f is not None)
    for head in [n for n in layer_of if n not in followed and isinstance(n.args[2], int)]:
        chain = [head]
        while followers.get(chain[-1]) is not None:
            chain.append(followers[chain[-1]])
        if len(chain) < 2:
            continue
        parent, seeds, _, replace = head.args
        with gm.graph.inserting_before(head):
            layers = gm.graph.call_function(
                sample_layer_chain, (parent, seeds, [n.args[2] for n in chain], replace))
            for l, fused in enumerate(chain):
                layer = gm.graph.call_function(operator.getitem, (layers, l))
                relabel, data = layer_of[fused]
                relabel.replace_all_uses_with(gm.graph.call_function(operator.getitem, (layer, 0)))
                if data:
                    values = gm.graph.call_function(operator.getitem, (layer, 1))
                    for query in data:
                        query.replace_all_uses_with(values)
        # later layers first: each one's seeds are a use of the layer before
        for fused in reversed(chain):
            relabel, data = layer_of[fused]
            for node in data + [relabel, fused]:
                gm.graph.erase_node(node)
    return dead_code(gm)


def layerwise_block(graph, seeds, fanout):
    """(tuple of `Graph::Relabel`, edge data) of one layer of a layer-wise sampler: what
    the chain below returns under the same seed.  A root graph takes the layer in one call of
    the C++ layer; its block has no edge-id map, the values come in the order of its edges."""
    parts = graph._CAPI_LayerwiseBlockIfFused(seeds, int(fanout))
    if parts:
        frontier, indptr, rows, values = parts
        return (frontier, frontier.numel(), seeds.numel(), indptr, rows, None, "csc"), values
    U = graph._CAPI_Slicing(seeds, 0, _CSC, _COO, False)
    prob = U._CAPI_Sum(1, 2, _CSR)
    picked = torch.ops.gs_ops.list_sampling_with_probs(U._CAPI_GetRows(), prob, fanout, False)[0]
    nodes = torch.cat((seeds, picked)).unique()
    sub = U._CAPI_Slicing(nodes, 1, _CSR, _COO, False)
    sub = sub._CAPI_Divide(prob[nodes], 1, _COO)._CAPI_Normalize(0, _CSC)
    return sub._CAPI_Relabel(), sub._CAPI_GetData("default")


def _only_users(node, *users):
    return set(node.users) == set(users)


def _match_layerwise_block(norm):
    """The nodes of one layer that ends in `norm` (a column normalisation), or None."""
    if not (_is_method(norm, ("_CAPI_Normalize", "_CAPI_normalize")) and norm.args[1:] == (0, _CSC)):
        return None
    relabel = [u for u in norm.users if _is_method(u, RELABEL) and u.args == (norm,)]
    data = [u for u in norm.users if _is_method(u, ("_CAPI_GetData", "_CAPI_get_data")) and
            u.args == (norm, "default") and not u.kwargs]
    if len(relabel) != 1 or len(relabel) + len(data) != len(norm.users):
        return None
    div = norm.args[0]
    if not (isinstance(div, fx.Node) and _is_method(div, ("_CAPI_Divide", "_CAPI_divide")) and
            len(div.args) == 4 and div.args[2:] == (1, _COO) and _only_users(div, norm)):
        return None
    sub, scale = div.args[0], div.args[1]
    if not (isinstance(sub, fx.Node) and _is_method(sub, SLICING) and len(sub.args) == 6 and
            sub.args[2:] == (1, _CSR, _COO, False) and _only_users(sub, div)):
        return None
    U, nodes = sub.args[0], sub.args[1]
    if not (isinstance(scale, fx.Node) and scale.op == "call_function" and
            scale.target is operator.getitem and scale.args[1] is nodes and _only_users(scale, div)):
        return None
    prob = scale.args[0]
    if not (isinstance(nodes, fx.Node) and nodes.op == "call_method" and nodes.target == "unique" and
            len(nodes.args) == 1 and not nodes.kwargs and _only_users(nodes, sub, scale)):
        return None
    cat = nodes.args[0]
    if not (isinstance(cat, fx.Node) and cat.op == "call_function" and cat.target is torch.cat and
            len(cat.args) == 1 and not cat.kwargs and isinstance(cat.args[0], (tuple, list)) and
            len(cat.args[0]) == 2 and _only_users(cat, nodes)):
        return None
    seeds, picked = cat.args[0]
    if not (isinstance(picked, fx.Node) and picked.op == "call_function" and
            picked.target is operator.getitem and picked.args[1] == 0 and _only_users(picked, cat)):
        return None
    pick = picked.args[0]
    if not (isinstance(pick, fx.Node) and pick.op == "call_function" and
            pick.target in _LIST_SAMPLING_WITH_PROBS and len(pick.args) == 4 and
            pick.args[1] is prob and isinstance(pick.args[2], int) and pick.args[3] is False and
            _only_users(pick, picked)):
        return None
    rows = pick.args[0]
    if not (isinstance(U, fx.Node) and _is_method(U, SLICING) and len(U.args) == 6 and
            U.args[1] is seeds and U.args[2:] == (0, _CSC, _COO, False)):
        return None
    if not (isinstance(rows, fx.Node) and _is_method(rows, ("_CAPI_GetRows", "_CAPI_get_rows")) and
            rows.args == (U,) and _only_users(rows, pick)):
        return None
    if not (isinstance(prob, fx.Node) and _is_method(prob, ("_CAPI_Sum", "_CAPI_sum")) and
            prob.args == (U, 1, 2, _CSR) and _only_users(prob, pick, scale)):
        return None
    if not _only_users(U, prob, rows, sub):
        return None
    # users first, so that the nodes can be erased in this order
    return {"relabel": relabel[0], "data": data, "graph": U.args[0], "seeds": seeds,
            "fanout": pick.args[2],
            "nodes": [norm, div, scale, sub, nodes, cat, picked, pick, rows, prob, U]}


def _list_sampling_targets():
    names = ("list_sampling_with_probs", "_CAPI_ListSamplingWithProbs")
    found = []
    for name in names:
        try:
            packet = getattr(torch.ops.gs_ops, name)
        except (AttributeError, RuntimeError):
            continue
        found.append(packet)
        found.extend(getattr(packet, o) for o in packet.overloads())
    return tuple(found)


_LIST_SAMPLING_WITH_PROBS = ()


def fuse_layerwise_block(gm: fx.GraphModule) -> fx.GraphModule:
    global _LIST_SAMPLING_WITH_PROBS
    if not _LIST_SAMPLING_WITH_PROBS:
        _LIST_SAMPLING_WITH_PROBS = _list_sampling_targets()
    for norm in list(gm.graph.nodes):
        layer = _match_layerwise_block(norm)
        if layer is None:
            continue
        with gm.graph.inserting_before(layer["relabel"]):
            fused = gm.graph.call_function(layerwise_block,
                                           (layer["graph"], layer["seeds"], layer["fanout"]))
            layer["relabel"].replace_all_uses_with(gm.graph.call_function(operator.getitem, (fused, 0)))
            if layer["data"]:
                values = gm.graph.call_function(operator.getitem, (fused, 1))
                for query in layer["data"]:
                    query.replace_all_uses_with(values)
        for node in layer["data"] + [layer["relabel"]] + layer["nodes"]:
            gm.graph.erase_node(node)
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


DEFAULT = (merge_relabel_and_all_indices, fuse_slicing_and_sampling, chain_sampled_layers,
           fuse_layerwise_block, common_subexpressions, dead_code)
