#!/usr/bin/env python3
"""GraphSAGE minibatch sampling benchmark (one MI355X).

One step = one [15,10,5] minibatch over 1024 fresh seed nodes on a synthetic R-MAT graph
resident in HBM: per layer a fused column slice + uniform sample without replacement (the
graph's fp32 edge weights follow the samples), then unique / relabel of (seeds, sampled rows);
the frontier feeds the next layer.  The headline graph is the large configuration: 111 M nodes /
1.6 B edges with int64 offsets, int32 ids and fp32 edge weights attached.  The timed step is ONE
call of the drop-in Graph class, _CAPI_SampleLayers, which does what the loop of the reference's
examples does (examples/graphsage/batching.py:125-138) with every layer queued on the device
and the sizes collected once; the same minibatches through the per-layer calls of that loop
(_CAPI_FusedColumnwiseSlicingSampling + _CAPI_Relabel, the drop-in pair) are reported beside it
(`per_layer_api`), as are the adjacency alone, u_dot_v on every block, and -- on the 2.45 M-node
graph -- the reference's own Algorithm R, the unfused operators, the super-batch operators, the
pool of sampler threads and 64-bit ids; then the layer-wise sampler (LADIES) and the walks at
the sizes of their configurations.  Everything reaches the HIP kernels of libgs_hip.so through
its C ABI.

Prints ONE JSON line: sampled edges per second, the roofline of the launch site that holds the
most GPU time (timed with hipEvents on the launch stream by the library's own hook), the
roofline of the whole step, and a host-core baseline of the same minibatches.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (nodes, edges, index dtype)
    "rmat-131k-2.1M": (1 << 17, 1 << 21, "int32"),
    "rmat-2.45M-124M": (2_450_000, 124_000_000, "int32"),
    "rmat-111M-1.6B": (111_000_000, 1_600_000_000, "int32"),
}
LARGE = "rmat-111M-1.6B"
SAGE = "rmat-2.45M-124M"
FANOUTS = (15, 10, 5)
BATCH = 1024
FEATURE_DIM = 64
HBM_PEAK_GBS = 8000.0
SUPER = 64  # minibatches per super-batch call


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=LARGE, choices=sorted(WORKLOADS))
    ap.add_argument("--no-weights", action="store_true",
                    help="the headline graph as an adjacency alone (no edge data follows the samples)")
    ap.add_argument("--cpu-steps", type=int, default=-1,
                    help="minibatches timed for the host-core baseline (-1: sized to ~15 s)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the timed step and its roofline: for profiling the step alone")
    ap.add_argument("--api", default="layers", choices=("layers", "loop"),
                    help="what --headline-only runs: the one-call minibatch or the per-layer calls")
    ap.add_argument("--legs", default="config_2,ladies,walks",
                    help="which legs follow the headline (comma-separated; empty: none)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain device copy of 496 MB (a kernel of known traffic to "
                         "scale hardware byte counters by)")
    return ap.parse_args()


class KernelTimer:
    """The library's launch-site timing hook: hipEvent pairs around every launch of
    one named site, recorded on the stream the kernel is launched on."""

    def __init__(self, lib):
        self.lib = lib
        lib.gs_profile_enable.argtypes = [ctypes.c_char_p]
        lib.gs_profile_collect.argtypes = [ctypes.POINTER(ctypes.c_double),
                                           ctypes.POINTER(ctypes.c_int64),
                                           ctypes.POINTER(ctypes.c_double), ctypes.c_int64]

    def enable(self, site, every=1):
        assert self.lib.gs_profile_stride(int(every)) == 0
        assert self.lib.gs_profile_enable(site.encode() if site else None) == 0

    def collect(self):
        total = ctypes.c_double()
        n = ctypes.c_int64()
        per = (ctypes.c_double * 4096)()
        assert self.lib.gs_profile_collect(ctypes.byref(total), ctypes.byref(n), per, 4096) == 0
        return total.value, n.value, list(per[:n.value])


class Ctx:
    """What every leg needs: modules, the device, the timing hook, the oracle (None: --no-cpu)."""

    def __init__(self, torch, np, gs, capi, rmat, timer, O, dev, args):
        self.torch, self.np, self.gs, self.capi, self.rmat = torch, np, gs, capi, rmat
        self.timer, self.O, self.dev, self.args = timer, O, dev, args


# ---------------------------------------------------------------------------------------
# Launch sites of one minibatch step and the bytes each launch must move at the least
# (b = bytes per id; S seeds, E sampled edges, M = S + E items, U distinct ids of a layer;
# w = 8 when the graph carries edge data -- the sample's weight read and written --, else 0):
#   sample        per seed   column id b + two offsets 16 + output offset 8
#                 per edge   neighbour gather b + sampled id store b + w (no select_index: the
#                            host layer asks for none, the weights are gathered in the launch)
#   insert        per item   one 8-byte slot read-modify-write 16 + slot index 4 (+ the id b when
#                            it is a launch of its own and reads the ids again)
#   compact       per item   slot index 4 + slot word 8 + first index set aside 8, per U id b
#   finish        per edge   first index 8 + prefix 8 + renamed id b; per item slot emptied 8;
#                 per seed   offsets copy 16
#   rank+rename   per item   slot index 4 + slot word 8 + distance 2, per edge renamed id b,
#                            per U id b; per item of the layer before, slot emptied 8 + index 4
#   sweep         per item   slot index 4 + slot emptied 8
def sample_bytes(b, w, S, E, U):
    return S * (b + 24) + E * (2 * b + w)


def insert_bytes(b, w, S, E, U):
    return (S + E) * (b + 20)


def compact_bytes(b, w, S, E, U):
    return (S + E) * 20 + U * b


def finish_bytes(b, w, S, E, U):
    return E * (16 + b) + (S + E) * 8 + S * 16


def layer_sample_bytes(b, w, S, E, U):
    return sample_bytes(b, w, S, E, U) + (S + E) * 20


def layer_relabel_bytes(b, w, S, E, U):
    return (S + E) * 14 + E * b + U * b


def sweep_bytes(b, w, S, E, U):
    return (S + E) * 12


SITE_BYTES = {
    "layers": {"layer_sample": layer_sample_bytes, "layer_relabel": layer_relabel_bytes,
               "layer_sweep": sweep_bytes},
    "loop": {"sample_fused": sample_bytes, "table_insert": insert_bytes,
             "unique_compact": compact_bytes, "unique_finish": finish_bytes},
}
SITE_KERNEL = {
    "layer_sample": "sample_group_kernel<linked> (column slice + count + scan + uniform sample + "
                    "edge-weight gather + hash insert of seeds and sampled ids in one launch, all "
                    "three layers)",
    "layer_relabel": "rank_linked_kernel (first-occurrence flags, their scan, frontier and renamed "
                     "ids in one launch; empties the table of the layer before)",
    "layer_sweep": "layer_sweep_kernel (empties the last layer's table slots)",
    "sample_fused": "sample_group_kernel (column slice + count + scan + uniform sample in one launch)",
    "table_insert": "table_insert_kernel (hash insert of seeds + sampled rows)",
    "unique_compact": "compact_kernel (first-occurrence flags, their scan, frontier)",
    "unique_finish": "finish_linked_kernel (renamed ids, offsets copy, table slots emptied)",
}
LAUNCHES_PER_STEP = {"layer_sweep": 1}


def step_bytes(sizes, weighted):
    """Bytes of one fused GraphSAGE minibatch by the per-unit figures of the scope table this
    build follows (reference widths: 8-byte ids): per layer 32 S + 16 E for slice + sample,
    64 (S + E) + 32 E + 16 U for unique + relabel, and 8 E for the edge data of the samples
    (4 read, 4 written) when the graph has any; no table-clearing term, the table here is
    emptied slot by slot."""
    return sum(32 * S + 16 * E + 64 * (S + E) + 32 * E + 16 * U + (8 * E if weighted else 0)
               for S, E, U in sizes)


def empty_pair_us(torch):
    """What an event pair with nothing between reads on the current stream: the share of
    avg_launch_us that is the two records' own (a kernel trace does not have it)."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(20)]
    torch.cuda.synchronize()
    for a, b in pairs:
        a.record()
        b.record()
    torch.cuda.synchronize()
    reads = sorted(a.elapsed_time(b) for a, b in pairs)
    return reads[len(reads) // 2] * 1e3


def traffic_from_profile(site, workload):
    """HBM bytes per launch of `site` as the hardware counters gave them (FETCH_SIZE and
    WRITE_SIZE passes scaled by a device copy of known size): the line
    `traffic_bytes_per_launch = N` of profiles/<site>_<workload>_hbm_counters.txt, or None when
    no such summary has been made for this site and workload."""
    path = os.path.join(ROOT, "profiles", "%s_%s_hbm_counters.txt" % (site, workload))
    try:
        m = re.search(r"^traffic_bytes_per_launch\s*=\s*(\d+)", open(path).read(), re.M)
    except OSError:
        return None
    return int(m.group(1)) if m else None


# ---------------------------------------------------------------------------------------
def minibatch_layers(graph, seeds):
    """One minibatch as ONE call of the drop-in Graph class: every layer queued with no host
    read in between.  Returns (#sampled edges, per-layer (S, E, U), flat result list: per layer
    frontier, offsets, renamed ids and -- on a graph with edge data -- the samples' data)."""
    parts = graph._CAPI_SampleLayers(seeds, list(FANOUTS), False)
    per = len(parts) // len(FANOUTS)
    total, sizes, S = 0, [], seeds.numel()
    for l in range(len(FANOUTS)):
        U, E = parts[per * l].numel(), parts[per * l + 2].numel()
        sizes.append((S, E, U))
        total += E
        S = U
    return total, sizes, parts


def minibatch_loop(graph, seeds, with_data=False):
    """The same minibatch through exactly the calls of the reference's examples
    (examples/graphsage/batching.py:125-138): per layer
    _CAPI_FusedColumnwiseSlicingSampling(seeds, fanout, False) then _CAPI_Relabel() (and, on a
    graph with edge data, _CAPI_GetData of the sample for the block's weights)."""
    total, sizes, parts = 0, [], []
    for k in FANOUTS:
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
        frontier, num_src, num_dst, indptr, indices, e_ids, fmt = sub._CAPI_Relabel()
        E = indices.numel()
        sizes.append((num_dst, E, num_src))
        parts += [frontier, indptr, indices]
        if with_data:
            parts.append(sub._CAPI_GetData("default"))
        total += E
        seeds = frontier
    return total, sizes, parts


def minibatch_nonfused(graph, seeds):
    """The same minibatch through the unfused operators of the Matrix API (A[:, seeds] ->
    columnwise_sampling -> relabel; python/gs/matrix_api/matrix.py:66-84 of the reference):
    _CAPI_Slicing(seeds, 0, _CSC, _COO) materialises every neighbour of the seeds first."""
    total = 0
    for k in FANOUTS:
        sliced = graph._CAPI_Slicing(seeds, 0, 2, 1, False)
        sub = sliced._CAPI_Sampling(0, k, False, 2, 1)
        frontier, num_src, num_dst, row, col, e_ids, fmt = sub._CAPI_Relabel()
        total += row.numel()
        seeds = frontier
    return total


def super_batch(torch, graph, seed_sets):
    """B minibatches sampled as ONE call per layer, the reference's own answer to launch
    latency (examples/graphsage/batching.py:59-88): fused sampling over the concatenated seeds,
    GetBatchCSC, BatchCSRRelabel (one relabel per minibatch, done in one pass), then the splits
    into per-minibatch blocks.  Returns (#sampled edges, per-layer (S, E, U) over all batches)."""
    seeds = torch.cat(seed_sets)
    ptr = torch.arange(len(seed_sets) + 1, dtype=torch.int64, device=seeds.device) * BATCH
    total, sizes = 0, []
    ops = torch.ops.gs_ops
    for k in FANOUTS:
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
        indptr, indices, indices_ptr = sub._CAPI_GetBatchCSC(ptr)
        uni, uni_ptr, rel, indices_ptr = ops.BatchCSRRelabel(seeds, ptr, indices, indices_ptr)
        blocks = (ops.SplitByOffset(uni, uni_ptr), ops.IndptrSplitByOffset(indptr, ptr),
                  ops.SplitByOffset(rel, indices_ptr))
        sizes.append((seeds.numel(), indices.numel(), uni.numel()))
        total += indices.numel()
        seeds, ptr = uni, uni_ptr
    return total, sizes, blocks


def cpu_minibatch(O, np, indptr, indices, weights, seeds, step):
    """One minibatch by the oracle on host arrays: per layer sample, the samples' weights (when
    the graph has any), unique + relabel."""
    total = 0
    for layer, k in enumerate(FANOUTS):
        sub_indptr, _, sub_indices, sel = O.sample_uniform(indptr, indices, seeds, k, False,
                                                           seed=step * len(FANOUTS) + layer,
                                                           with_coo=False)
        if weights is not None:
            weights[sel]
        frontier, _ = O.relabel([seeds, sub_indices], [sub_indices])
        total += int(sub_indptr[-1])
        seeds = frontier
    return total, seeds


def columns_of(torch, indptr, indices, cols):
    """(offsets, neighbour ids, positions in `indices`) of the columns `cols`, cut out of the
    graph with plain torch indexing (no library kernel): what the checker below hands to the
    oracle."""
    starts = indptr[cols]
    deg = indptr[cols + 1] - starts
    offsets = torch.zeros(cols.numel() + 1, dtype=torch.int64, device=indptr.device)
    torch.cumsum(deg, 0, out=offsets[1:])
    total = int(offsets[-1])
    owner = torch.repeat_interleave(torch.arange(cols.numel(), device=indptr.device), deg,
                                    output_size=total)
    pos = torch.arange(total, device=indptr.device) - offsets[owner] + starts[owner]
    return offsets, indices[pos], pos


def check_against_oracle(torch, np, O, indptr, indices, weights, seeds, first_seed, parts):
    """The checker: the minibatch `parts` ([frontier, offsets, renamed ids(, data)] per layer)
    against the oracle run layer by layer with the same draws.  The oracle gets each layer's
    columns as a small graph of their own (the draws of a column depend on its place in the
    call, not on its id), so a graph of any size is checked without a host copy of it; the
    samples' edge data must equal weights[select_index], the oracle's positions taken back to
    the whole graph's."""
    per = len(parts) // len(FANOUTS)
    cols = seeds.long()
    for l, k in enumerate(FANOUTS):
        sub_ptr, sub_idx, pos = columns_of(torch, indptr, indices, cols)
        h_ptr, h_idx = sub_ptr.cpu().numpy(), sub_idx.cpu().numpy().astype(np.int64)
        h_cols = cols.cpu().numpy()
        w_ptr, _, w_rows, w_sel = O.sample_uniform(h_ptr, h_idx, np.arange(h_cols.size, dtype=np.int64),
                                                   k, False, seed=first_seed + l, with_coo=False)
        w_frontier, (w_renamed,) = O.relabel([h_cols, w_rows], [w_rows])
        got = [p.cpu().numpy().astype(np.int64) for p in parts[per * l:per * l + 3]]
        if not (np.array_equal(got[0], w_frontier) and np.array_equal(got[1], w_ptr)
                and np.array_equal(got[2], w_renamed)):
            return False
        if weights is not None:
            want = weights[pos[torch.from_numpy(w_sel).to(indptr.device)]]
            if per != 4 or not torch.equal(parts[per * l + 3], want):
                return False
        cols = torch.from_numpy(w_frontier).to(indptr.device)
    return True


def saturated(torch, graph, timer, nodes, idt, dev, b):
    """The sampler launch at a size that fills the chip (4M seed columns drawn with
    repetition, fanout 10): what the kernel reaches once launch latency is amortised."""
    S = 1 << 22
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    cols = torch.randint(0, nodes, (S,), generator=gen, device=dev).to(idt)
    timer.enable("sample_fused")
    E = 0
    for _ in range(4):
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(cols, 10, False)
        E = sub._CAPI_GetNumEdges()
    torch.cuda.synchronize()
    ms, n, per = timer.collect()
    timer.enable("")
    t = min(per[1:]) * 1e-3
    achieved = sample_bytes(b, 0, S, E, 0) / t / 1e9
    return {"kernel": "sample_row_lane_kernel (the one-launch sampler from 2^18 columns on: one row "
                      "per lane, edge-parallel fill)", "seeds": S, "fanout": 10, "sampled_edges": E,
            "launch_us": t * 1e6, "achieved": achieved, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS}


def leg(fn):
    """A secondary leg must not take the headline with it: when it raises, the traceback goes to
    stderr and the line carries {"error": ...} under the leg's key."""
    try:
        return fn()
    except Exception as e:  # noqa: BLE001 -- whatever it is, the headline is still worth printing
        import traceback
        traceback.print_exc()
        return {"error": "%s: %s" % (type(e).__name__, str(e)[:500])}


def timed(torch, fn, sets):
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    edges = 0
    for s in sets:
        edges += fn(s)
    torch.cuda.synchronize()
    return edges, time.perf_counter() - t1


# ---------------------------------------------------------------------------------------
def graphsage(cx, workload, weighted, with_features, full, cpu_budget):
    """The GraphSAGE leg on one graph: the timed step, its latency, the roofline of its dominant
    launch site and of the whole step, the host-core baseline; `full` adds the other ways of
    running the same minibatches.  Returns the keys of a bench line."""
    torch, np, gs, capi, O, dev, args = cx.torch, cx.np, cx.gs, cx.capi, cx.O, cx.dev, cx.args
    timer = cx.timer
    nodes, edges, idt = WORKLOADS[workload]
    idt = getattr(torch, idt)
    b = 4 if idt == torch.int32 else 8
    w = 8 if weighted else 0
    api = args.api if args.headline_only else "layers"
    step_fn = {"layers": minibatch_layers,
               "loop": lambda g, s: minibatch_loop(g, s, weighted)}[api]

    t0 = time.perf_counter()
    indptr, indices = cx.rmat.rmat_csc(nodes, edges, seed=0, device=dev, index_dtype=idt)
    gen = torch.Generator(device=dev)
    weights = None
    if weighted:
        gen.manual_seed(1)
        weights = 1.0 - torch.rand(edges, generator=gen, device=dev)  # ~U(0, 1]
    torch.cuda.synchronize()
    gen_s = time.perf_counter() - t0

    graph = gs.Graph(False)
    graph._CAPI_LoadCSC(indptr, indices)
    if weighted:
        graph._CAPI_SetData(weights)
    if args.calibration_copy:
        src = torch.empty(124_000_000, dtype=torch.int32, device=dev)
        torch.empty_like(src).copy_(src)
        torch.cuda.synchronize()
        del src

    gen.manual_seed(2)

    def fresh_seeds():
        return torch.randperm(nodes, generator=gen, device=dev)[:BATCH].to(idt)

    seed_sets = [fresh_seeds() for _ in range(args.warmup + args.steps)]
    timed_sets = seed_sets[args.warmup:]
    first_seed = args.warmup * len(FANOUTS)
    torch.cuda.synchronize()

    # the Graph API draws seed, seed+1, ... per sampled layer: 3 per step
    torch.ops.gs_ops._CAPI_SetSeed(0)
    for i in range(args.warmup):
        step_fn(graph, seed_sets[i])
    torch.cuda.synchronize()

    # which launch site holds the most GPU time: one untimed step per site
    site_ms = {}
    for site in SITE_BYTES[api]:
        timer.enable(site)
        step_fn(graph, seed_sets[0])
        torch.cuda.synchronize()
        site_ms[site] = timer.collect()[0]
    dominant = max(site_ms, key=lambda k: site_ms[k])
    per_step = LAUNCHES_PER_STEP.get(dominant, len(FANOUTS))

    torch.ops.gs_ops._CAPI_SetSeed(first_seed)
    # every 7th launch of the dominant site is bracketed by an event pair: with three
    # launches per step that visits the three layers in turn, and keeps the pairs' own
    # queue time (about 6 us each, as long as the kernel) mostly out of the measurement
    timer.enable(dominant, every=7 if per_step == len(FANOUTS) else 1)
    sampled = 0
    first = None
    algo_bytes = 0
    whole_step_bytes = 0
    torch.cuda.synchronize()
    t_begin = time.perf_counter()
    all_sizes = []
    for s in timed_sets:
        # a step ends when the host holds every tensor size of the minibatch (the call hands
        # back tensors of their final lengths); nothing else synchronises inside the loop,
        # and the byte counts are made from the sizes afterwards
        n, sizes, parts = step_fn(graph, s)
        sampled += n
        all_sizes.append(sizes)
        if first is None:
            first = (n, parts)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_begin
    k_ms, k_launches, _ = timer.collect()
    timer.enable("")
    layer_sizes = all_sizes[-1]
    for sizes in all_sizes:
        if per_step == 1:
            algo_bytes += SITE_BYTES[api][dominant](b, w, *sizes[-1])
        else:
            algo_bytes += sum(SITE_BYTES[api][dominant](b, w, *z) for z in sizes)
        whole_step_bytes += step_bytes(sizes, weighted)

    # the checker: step 0 of the timed region must agree with the oracle bit for bit
    checked = None
    if O is not None:
        if not check_against_oracle(torch, np, O, indptr, indices, weights, timed_sets[0],
                                    first_seed, first[1]):
            print("bench.py: GPU minibatch on %s differs from the oracle on the same seeds and "
                  "draws" % workload, file=sys.stderr)
            sys.exit(1)
        checked = ("step 0 of the timed region: frontier, offsets and renamed ids of every layer "
                   "bit for bit against the oracle" +
                   (", the samples' weights equal to weights[select_index]" if weighted else ""))

    # latency of one minibatch with the device drained before and after it (untimed pass over
    # the same seed sets; a different quantity from ms_per_step, whose steps run back to back)
    lat = []
    for s in timed_sets:
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        step_fn(graph, s)
        torch.cuda.synchronize()
        lat.append(time.perf_counter() - t1)
    lat.sort()
    p50 = lat[len(lat) // 2] * 1e3
    p90 = lat[min(len(lat) - 1, int(len(lat) * 0.9))] * 1e3

    out = {
        "value": sampled / elapsed,
        "ms_per_step": elapsed / args.steps * 1e3,
        "p50_ms": p50,
        "p90_ms": p90,
        "dtype": "int32" if idt == torch.int32 else "int64",
        "config": {"workload": workload, "nodes": nodes, "edges": edges, "batch": BATCH,
                   "fanouts": list(FANOUTS),
                   "edge_weights": "fp32 ~U(0,1], attached with _CAPI_SetData: every layer returns "
                                   "its samples' weights" if weighted else None,
                   "last_step_layers_S_E_U": layer_sizes,
                   "graph_build_s": round(gen_s, 2),
                   "api": "gs_classes.Graph._CAPI_SampleLayers (one call per minibatch; an entry the "
                          "reference does not have -- `per_layer_api` is the reference's own call pair)"
                          if api == "layers" else
                          "gs_classes.Graph._CAPI_FusedColumnwiseSlicingSampling + _CAPI_Relabel per layer"},
        "checked": checked,
    }
    step_gbs = whole_step_bytes / elapsed / 1e9
    out["step_roofline"] = {
        "bound": "hbm", "achieved": step_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": step_gbs / HBM_PEAK_GBS, "bytes_per_step": whole_step_bytes / args.steps,
        "what": "per layer 32 S + 16 E (slice + sample) + 64 (S + E) + 32 E + 16 U (unique + "
                "relabel)%s, reference id widths, over ms_per_step"
                % (" + 8 E (the samples' weights)" if weighted else "")}
    out["roofline"] = None
    if k_launches:
        avg_s = k_ms * 1e-3 / k_launches
        bytes_per_launch = algo_bytes / (per_step * args.steps)
        achieved = bytes_per_launch / avg_s / 1e9
        out["roofline"] = {
            "bound": "hbm",
            "kernel": SITE_KERNEL[dominant],
            "site": dominant,
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic_from_profile(dominant, workload),
            "traffic_source": "profiles/%s_%s_hbm_counters.txt" % (dominant, workload),
            "launches": per_step * args.steps,
            "launches_timed": k_launches,
            "avg_launch_us": avg_s * 1e6,
            "empty_event_pair_us": empty_pair_us(torch),
            "algorithmic_bytes_per_launch": bytes_per_launch,
            "gpu_ms_per_step_by_site": {k: round(v, 4) for k, v in site_ms.items()},
        }

    extras = not args.headline_only
    ops = torch.ops.gs_ops

    # the per-layer calls of the reference's loop on the same seed sets and draws
    if extras:
        ops._CAPI_SetSeed(0)
        for s in seed_sets[:args.warmup]:
            minibatch_loop(graph, s, weighted)
        pl_e, pl_s = timed(torch, lambda s: minibatch_loop(graph, s, weighted)[0], timed_sets)
        ops._CAPI_SetSeed(first_seed)
        same = all(torch.equal(x, y)
                   for x, y in zip(minibatch_loop(graph, timed_sets[0], weighted)[2], first[1]))
        out["per_layer_api"] = {
            "ms_per_step": pl_s / args.steps * 1e3, "value": pl_e / pl_s,
            "identical_to_headline_step0": bool(same),
            "what": "the drop-in call pair: _CAPI_FusedColumnwiseSlicingSampling + _CAPI_Relabel "
                    "per layer (examples/graphsage/batching.py:125-138)%s: one host wait per layer"
                    % (" + _CAPI_GetData of every sample" if weighted else "")}

    # the same minibatches with the next one queued before this one is collected
    if extras:
        per = 4 if weighted else 3

        def pipelined(sets):
            edges, ahead = 0, graph._CAPI_QueueSampleLayers(sets[0], list(FANOUTS), False)
            for nxt in list(sets[1:]) + [None]:
                following = (graph._CAPI_QueueSampleLayers(nxt, list(FANOUTS), False)
                             if nxt is not None else None)
                parts = ahead.collect()
                edges += sum(parts[per * l + 2].numel() for l in range(len(FANOUTS)))
                ahead = following
            return edges

        ops._CAPI_SetSeed(0)
        pipelined(seed_sets[:args.warmup])
        ops._CAPI_SetSeed(first_seed)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        q_e = pipelined(timed_sets)
        torch.cuda.synchronize()
        q_s = time.perf_counter() - t1
        out["queued_ahead"] = {
            "ms_per_step": q_s / args.steps * 1e3, "value": q_e / q_s,
            "same_edges_as_headline": bool(q_e == sampled),
            "what": "_CAPI_QueueSampleLayers of minibatch i + 1 before .collect() of minibatch i (one "
                    "thread, one stream): the same minibatches, the stream does not wait for the "
                    "host between them"}

    # the same graph without its weights / with them, whichever the headline is not
    if extras and full != "config2":
        other = gs.Graph(False)
        other._CAPI_LoadCSC(indptr, indices)
        ops._CAPI_SetSeed(0)
        for s in seed_sets[:args.warmup]:
            minibatch_layers(other, s)
        a_e, a_s = timed(torch, lambda s: minibatch_layers(other, s)[0], timed_sets)
        out["adjacency_only"] = {
            "ms_per_step": a_s / args.steps * 1e3, "value": a_e / a_s,
            "what": "the timed minibatches on the same graph loaded without edge data (as the "
                    "reference's GraphSAGE examples load it): nothing follows the samples"}
        del other

    # the throughput form on the same graph: 64 minibatches per call
    if extras and full != "config2":
        out["super_batch"] = leg(lambda: super_batch_leg(torch, graph, timer, fresh_seeds, b,
                                                         weighted, workload))

    # u_dot_v with 64-d fp32 node features on every block (the large configuration's second half)
    if extras and with_features:
        gen.manual_seed(3)
        features = torch.rand(nodes, FEATURE_DIM, generator=gen, device=dev) - 0.5
        per = 4 if weighted else 3

        def dots(parts):
            outs = []
            for l in range(len(FANOUTS)):
                frontier, offsets, renamed = parts[per * l:per * l + 3]
                h = features.index_select(0, frontier)  # source features; seeds come first
                o = torch.empty(renamed.numel(), 1, device=dev)
                capi.sddmm_csc("dot", offsets, renamed, None, None, h, h[:offsets.numel() - 1], o,
                               0, 2, FEATURE_DIM, FEATURE_DIM, 1, FEATURE_DIM)
                outs.append(o)
            return outs

        def step_dots(seeds):
            n, sizes, parts = minibatch_layers(graph, seeds)
            dots(parts)
            return n

        for s in seed_sets[:args.warmup]:
            step_dots(s)
        ok = True
        if O is not None:
            for l, o in enumerate(dots(first[1])):
                frontier, offsets, renamed = first[1][per * l:per * l + 3]
                h = features[frontier.long()]
                col = torch.repeat_interleave(torch.arange(offsets.numel() - 1, device=dev),
                                              offsets[1:] - offsets[:-1])
                want = (h[renamed.long()] * h[col]).sum(-1, keepdim=True)
                ok = ok and bool(torch.allclose(o, want, rtol=1e-5, atol=1e-6))
            if not ok:
                print("bench.py: u_dot_v on %s differs from the torch gather-and-dot" % workload,
                      file=sys.stderr)
                sys.exit(1)
        ops._CAPI_SetSeed(first_seed)
        d_e, d_s = timed(torch, step_dots, timed_sets)
        timer.enable("sddmm_dot")
        for s in timed_sets[:20]:
            step_dots(s)
        torch.cuda.synchronize()
        d_ms, d_n, _ = timer.collect()
        timer.enable("")
        # dot of two 64-float rows per edge: 2 x 256 B of features + 12 B of ids + 4 B out
        dot_bytes = sum(E for _, E, _ in layer_sizes) / len(FANOUTS) * (2 * 4 * FEATURE_DIM + 12 + 4)
        dot_gbs = dot_bytes / (d_ms * 1e-3 / d_n) / 1e9 if d_n else None
        out["with_u_dot_v"] = {
            "feature_dim": FEATURE_DIM, "ms_per_step": d_s / args.steps * 1e3, "value": d_e / d_s,
            "checked": "step 0: u_dot_v of every block at 1e-5 against a torch gather-and-dot"
                       if O is not None else None,
            "sddmm_dot": {"avg_launch_us": d_ms * 1e3 / d_n if d_n else None, "achieved": dot_gbs,
                          "unit": "GB/s", "frac": dot_gbs / HBM_PEAK_GBS if dot_gbs else None,
                          "what": "u_dot_v launches of the three blocks"},
            "what": "the timed step, then features[frontier] and gs_sddmm_csc(dot) on each of the "
                    "three blocks (AS-GCN-style attention scores)"}
        del features

    if extras and full == "config2":
        # the same graph with fp32 edge weights attached (the layer-wise configuration's graph)
        gen.manual_seed(1)
        wts = 1.0 - torch.rand(edges, generator=gen, device=dev)
        gw = gs.Graph(False)
        gw._CAPI_LoadCSC(indptr, indices)
        gw._CAPI_SetData(wts)
        for s in seed_sets[:args.warmup]:
            minibatch_layers(gw, s)
        ops._CAPI_SetSeed(first_seed)
        w_first = minibatch_layers(gw, timed_sets[0])[2]
        if O is not None and not check_against_oracle(torch, np, O, indptr, indices, wts,
                                                      timed_sets[0], first_seed, w_first):
            print("bench.py: the weighted minibatch on %s differs from the oracle" % workload,
                  file=sys.stderr)
            sys.exit(1)
        w_e, w_s = timed(torch, lambda s: minibatch_layers(gw, s)[0], timed_sets)
        out["with_edge_weights"] = {
            "ms_per_step": w_s / args.steps * 1e3, "value": w_e / w_s,
            "what": "the timed minibatches on the same graph with fp32 edge weights attached: every "
                    "layer also returns its samples' weights (step 0 checked against the oracle)"}
        del gw, wts, w_first

        # the reference's own selection algorithm (Algorithm R, src/cuda/sampling.cu:70-92) on
        # the same seed sets: the count / reservoir / gather kernels instead of the one-launch sampler
        ops._CAPI_SetSampleAlgo(1)
        rs_steps = min(args.steps, 50)
        for s in seed_sets[:3]:
            minibatch_loop(graph, s)
        rs_e, rs_s = timed(torch, lambda s: minibatch_loop(graph, s)[0], timed_sets[:rs_steps])
        ops._CAPI_SetSampleAlgo(0)
        out["reservoir_mode"] = {
            "ms_per_step": rs_s / rs_steps * 1e3, "value": rs_e / rs_s, "steps": rs_steps,
            "what": "GS_SAMPLE_RESERVOIR through the per-layer calls: deg - fanout draws per "
                    "column, output in slot order, bit-exact against the reference's "
                    "draw sequence under replay"}

        # the unfused operator sequence on the same seed sets
        nf_steps = min(args.steps, 50)
        for s in seed_sets[:3]:
            minibatch_nonfused(graph, s)
        nf_e, nf_s = timed(torch, lambda s: minibatch_nonfused(graph, s), timed_sets[:nf_steps])
        out["unfused_path"] = {
            "ms_per_step": nf_s / nf_steps * 1e3, "value": nf_e / nf_s, "steps": nf_steps,
            "what": "Slicing -> Sampling -> Relabel per layer instead of the fused sampler"}

        out["super_batch"] = leg(lambda: super_batch_leg(torch, graph, timer, fresh_seeds, b, False,
                                                         workload))

        # the same minibatches with 64-bit ids, the reference's only id type
        if idt == torch.int32:
            graph64 = gs.Graph(False)
            graph64._CAPI_LoadCSC(indptr, indices.long())
            sets64 = [s.long() for s in seed_sets]
            for s in sets64[:args.warmup]:
                minibatch_layers(graph64, s)
            w_e, w_s = timed(torch, lambda s: minibatch_layers(graph64, s)[0], sets64[args.warmup:])
            out["int64_ids"] = {"ms_per_step": w_s / args.steps * 1e3, "value": w_e / w_s,
                                "what": "the timed minibatches on the same graph with int64 ids"}
            del graph64, sets64

        # the same again by the C++ layer's own pool of sampler threads (no interpreter in the
        # loop), 32 minibatches per call as a loader with that prefetch depth would ask for them
        DEPTH = 32
        # three sampler threads: a process has four hardware queues, one of them the null
        # stream's, and a fourth worker shares a queue with another one
        POOL = 3
        ops._CAPI_SampleBlocks(graph, seed_sets[:DEPTH], FANOUTS, False, POOL, 0)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        pool_edges = 0
        for c0 in range(0, len(timed_sets), DEPTH):
            res = ops._CAPI_SampleBlocks(graph, timed_sets[c0:c0 + DEPTH], FANOUTS, False, POOL,
                                         c0 * len(FANOUTS))
            pool_edges += sum(int(parts[3 * l + 2].numel()) for parts in res
                              for l in range(len(FANOUTS)))
            del res
        torch.cuda.synchronize()
        pool_s = time.perf_counter() - t1
        out["sampler_pool"] = {
            "workers": POOL, "minibatches_per_call": DEPTH,
            "ms_per_step": pool_s / len(timed_sets) * 1e3, "value": pool_edges / pool_s,
            "what": "the timed minibatches through gs_ops._CAPI_SampleBlocks: three host threads "
                    "of the C++ layer, one stream each, every minibatch queued whole"}
        out["roofline_saturated"] = saturated(torch, graph, timer, nodes, idt, dev, b)

    out["cpu_baseline"] = None
    if O is not None and cpu_budget > 0:
        # the whole graph on the host (the oracle's id type is int64), as a CPU sampler holds it
        t1 = time.perf_counter()
        h_indptr = indptr.cpu().numpy()
        h_indices = np.empty(edges, dtype=np.int64)
        CH = 1 << 28
        for lo in range(0, edges, CH):
            h_indices[lo:lo + CH] = indices[lo:lo + CH].cpu().numpy()
        h_weights = weights.cpu().numpy() if weighted else None
        copy_s = time.perf_counter() - t1
        h_seeds = [s.cpu().numpy().astype(np.int64) for s in timed_sets]
        n_ref, f_ref = cpu_minibatch(O, np, h_indptr, h_indices, h_weights, h_seeds[0], args.warmup)
        per = 4 if weighted else 3
        if n_ref != first[0] or not np.array_equal(f_ref, first[1][-per].cpu().numpy()):
            print("bench.py: GPU minibatch differs from the oracle on the same seeds and draws",
                  file=sys.stderr)
            sys.exit(1)
        t1 = time.perf_counter()
        done = 0
        cpu_edges = 0
        # passes over the timed seed sets (fresh draws every pass) until the budget is used up
        limit = args.cpu_steps if args.cpu_steps > 0 else 1 << 40
        while done < limit and (args.cpu_steps > 0 or time.perf_counter() - t1 < cpu_budget):
            cpu_edges += cpu_minibatch(O, np, h_indptr, h_indices, h_weights,
                                       h_seeds[done % len(h_seeds)], args.warmup + done)[0]
            done += 1
        cpu_s = time.perf_counter() - t1
        out["cpu_baseline"] = {
            "value": cpu_edges / cpu_s,
            "unit": "edges/s",
            "cores": O.num_threads(),
            "kind": "port",
            "sample": "%d minibatches in %.1f s: the timed seed sets (same seeds; the first pass "
                      "with the same draws) through the C oracle on a host copy of the whole graph "
                      "(made in %.1f s, not timed), OpenMP over rows%s; unique is "
                      "single-threaded; step 0 compared with the GPU result bit for bit"
                      % (done, cpu_s, copy_s,
                         ", the samples' weights gathered with numpy" if weighted else ""),
            "ms_per_step": cpu_s / done * 1e3,
        }
        del h_indptr, h_indices, h_weights
    del graph, indptr, indices, weights
    torch.cuda.empty_cache()
    return out


def super_batch_leg(torch, graph, timer, fresh_seeds, b, weighted, workload):
    """SUPER minibatches per call on seed sets of its own: what the kernels reach once a launch
    holds enough work for the chip."""
    per = 4 if weighted else 3
    # SUPER minibatches per call (a "super-batch"), on seed sets of its own: the C++ layer's
    # own loop (_CAPI_SampleLayersBatched), and the same flow written with the reference's
    # operators in Python (examples/graphsage/batching.py:59-88)
    groups = [[fresh_seeds() for _ in range(SUPER)] for _ in range(5)]

    def batched(grp):
        return graph._CAPI_SampleLayersBatched(grp, list(FANOUTS), False)

    def sizes_of(res):  # per layer (S, E, U) over all minibatches of a call
        sizes = [[sum(int(parts[per * l + j].numel()) for parts in res) for j in (1, 2, 0)]
                 for l in range(len(FANOUTS))]
        return [(S - len(res), E, U) for S, E, U in sizes]  # (offsets hold one entry more per batch)

    # warm-up with every call's result kept, as in the timed loop: the allocator then holds the
    # blocks of all of them (a fresh hipMalloc of a few hundred MB costs milliseconds)
    results = [batched(grp) for grp in groups]
    del results
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    results = [batched(grp) for grp in groups]  # a call ends with every minibatch's views made
    torch.cuda.synchronize()
    sb_s = time.perf_counter() - t1
    sb_sizes = sizes_of(results[-1])
    sb_edges = sum(sum(z[1] for z in sizes_of(res)) for res in results)
    del results
    # the same calls in two halves, super-batch i + 1 queued before super-batch i is collected:
    # the host's share of a call then runs while the stream works on the last layer
    def queued(grp):
        return graph._CAPI_QueueSampleLayersBatched(grp, list(FANOUTS), False)

    results = []
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    qa_groups = groups + groups  # (every call draws with fresh seeds: no call repeats another)
    ahead = queued(qa_groups[0])
    for grp in qa_groups[1:]:
        nxt = queued(grp)
        results.append(ahead.collect())
        ahead = nxt
    results.append(ahead.collect())
    torch.cuda.synchronize()
    qa_s = time.perf_counter() - t1
    qa_edges = sum(sum(z[1] for z in sizes_of(res)) for res in results)
    del results, ahead, nxt
    super_batch(torch, graph, groups[0])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    py_edges = 0
    for grp in groups:
        py_edges += super_batch(torch, graph, grp)[0]
    torch.cuda.synchronize()
    py_s = time.perf_counter() - t1
    sb_sites = {}
    for site in SUPER_SITES:
        timer.enable(site)
        batched(groups[0])
        torch.cuda.synchronize()
        ms, n, per_l = timer.collect()
        if n:
            sb_sites[site] = (ms, per_l)
    timer.enable("")
    sb_dom = max(sb_sites, key=lambda k: sb_sites[k][0])
    # the dominant site's largest launch (the third layer) against its bytes
    S3, E3, U3 = sb_sizes[-1]
    sb_bytes = SUPER_SITES[sb_dom](b, S3, E3, U3)
    if weighted and sb_dom == "sample_fused":
        sb_bytes += 8 * E3  # a weight read and written per sampled edge
    t3 = max(sb_sites[sb_dom][1]) * 1e-3
    gpu_ms = sum(v[0] for v in sb_sites.values())
    call_bytes = step_bytes(sb_sizes, weighted)
    out = {
        "minibatches_per_call": SUPER, "calls": len(groups),
        "ms_per_minibatch": sb_s / (len(groups) * SUPER) * 1e3, "value": sb_edges / sb_s,
        "ms_per_call": sb_s / len(groups) * 1e3,
        "layers_S_E_U": sb_sizes,
        "api": "gs_classes.Graph._CAPI_SampleLayersBatched (one call per super-batch)",
        "queued_ahead": {
            "calls": len(qa_groups), "ms_per_call": qa_s / len(qa_groups) * 1e3,
            "value": qa_edges / qa_s,
            "gpu_busy_frac": gpu_ms * 1e-3 / (qa_s / len(qa_groups)),
            "what": "_CAPI_QueueSampleLayersBatched of super-batch i + 1 before .collect() of "
                    "super-batch i (one thread, one stream)"},
        "through_python_ops": {
            "ms_per_minibatch": py_s / (len(groups) * SUPER) * 1e3, "value": py_edges / py_s,
            "what": "the same flow as _CAPI_FusedColumnwiseSlicingSampling + GetBatchCSC + "
                    "BatchCSRRelabel + SplitByOffset / IndptrSplitByOffset calls from Python"},
        "roofline": {"bound": "hbm", "kernel": sb_dom + " (third layer's launch)",
                     "achieved": sb_bytes / t3 / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": sb_bytes / t3 / 1e9 / HBM_PEAK_GBS, "launch_us": t3 * 1e6,
                     "algorithmic_bytes": sb_bytes,
                     # (the summaries were taken on the large graph with its edge weights and on
                     # config 2 without any)
                     "traffic": traffic_from_profile("super_batch", workload)
                     if sb_dom == "sample_fused" and weighted == (workload == LARGE) else None,
                     "traffic_source": "profiles/super_batch_%s_hbm_counters.txt" % workload,
                     "gpu_ms_by_site": {k: round(v[0], 4) for k, v in sb_sites.items()}},
        "step_roofline": {"bound": "hbm", "achieved": call_bytes / (sb_s / len(groups)) / 1e9,
                          "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": call_bytes / (sb_s / len(groups)) / 1e9 / HBM_PEAK_GBS,
                          "gpu_busy_frac": gpu_ms * 1e-3 / (sb_s / len(groups)),
                          "what": "the scope table's bytes of the whole call (as step_roofline) "
                                  "over its wall time; gpu_busy_frac = the sites' kernel time "
                                  "over the same"},
        "what": "fused sampling over the concatenated seeds + the batches' edge cuts + one relabel "
                "per minibatch in one pass (through hash classes and LDS tables from 2^19 items "
                "on) + per-minibatch views, 64 minibatches of 1024 seeds at once"}
    return out


def _sb_sample(b, S, E, U):
    return sample_bytes(b, 0, S, E, U)


# launch sites of the super-batch flow and the least bytes of each one's third-layer launch
# (M = S + E items; the binned relabel: count reads the ids, scatter reads them and writes an
# 8-byte record each, flag reads and rewrites the records and marks first occurrences, rank
# reads a byte and writes 16 bytes per 64 items, rename reads the records and a 16-byte entry
# each and writes the renamed ids and the frontier)
SUPER_SITES = {
    "sample_fused": _sb_sample,
    "bins_count": lambda b, S, E, U: (S + E) * b,
    "bins_scatter": lambda b, S, E, U: (S + E) * (b + 8),
    "bins_flag": lambda b, S, E, U: (S + E) * 16 + U,
    "bins_rank": lambda b, S, E, U: (S + E) * (1 + 0.25),
    "bins_rename": lambda b, S, E, U: (S + E) * (8 + 16) + E * b + U * b,
    "batch_init": lambda b, S, E, U: 4 * (S + E) * 8,            # 8-byte slots, 4 per item
    "batch_insert": lambda b, S, E, U: (S + E) * (b + 16 + 4 + 8),  # id, slot RMW, slot index, offsets
    "batch_compact": lambda b, S, E, U: (S + E) * 20 + U * b,
    "batch_finish": lambda b, S, E, U: E * (16 + b) + (S + E) * 4,
}


# ---------------------------------------------------------------------------------------
def make_ladies_sampler(torch, seen_probs=None):
    """`seen_probs` (a list): the run's row probabilities are appended to it, layer by layer,
    for the checker (they are sums by float atomics: another run's differ in the last bits)."""
    def ladies_sampler(A, seeds, fanouts):
        """The sampler of examples/ladies/ladies_raw.py:8-27, written against Matrix."""
        ret = []
        for fanout in fanouts:
            U = A[:, seeds]
            prob = U.sum(axis=1, powk=2)
            if seen_probs is not None:
                seen_probs.append(prob)
            selected, _ = torch.ops.gs_ops.list_sampling_with_probs(U.row_ids(unique=False), prob,
                                                                    fanout, False)
            nodes = torch.cat((seeds, selected)).unique()
            subU = U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0)
            seeds = subU.all_indices()
            ret.insert(0, subU.to_dgl_block())
        return seeds, ret
    return ladies_sampler


def cpu_ladies(O, np, indptr, indices, weights, seeds, picks, first_seed, probs=None):
    """The same sampler by the oracle on host arrays.  Returns per layer (frontier, renamed row,
    renamed col, normalised weights), outermost layer first like the sampler's blocks reversed.
    `probs` (a list, one per layer): row probabilities to pick by instead of the oracle's own
    (the checker hands in the device's, which differ from the oracle's in the last bits)."""
    N = indptr.size - 1
    layers = []
    for l, k in enumerate(picks):
        sp, coo, si, sel = O.slice_columns(indptr, indices, seeds)
        data = weights[sel]
        prob = O.coo_sum(si, None, data, 2, N)
        pick_by = prob if probs is None else probs[l]
        selected, _ = O.list_sample_weighted(np.arange(N, dtype=np.int64), pick_by, k,
                                             seed=first_seed + l)
        nodes = np.unique(np.concatenate([seeds, selected]))
        r_ip, r_col, r_perm = O.coo2csc(si, coo, N, False)
        s_ip, s_row, s_col, s_sel = O.slice_columns(r_ip, r_col, nodes)
        w_data = data[r_perm][s_sel]
        w_div = (w_data / prob[nodes][s_row]).astype(np.float32)
        col_sum = O.coo_sum(s_col, None, w_div, 1, seeds.size)
        w_norm = w_div / col_sum[s_col]
        # the block: Normalize(axis 0) left the graph with a CSC (stable sort of the row-ordered
        # edges by column), and Relabel takes the CSC when there is one (src/graph.cc:789-811):
        # frontier in the CSC's edge order, weights through its edge-id map
        c_ip, c_row, c_perm = O.coo2csc(s_col, s_row, seeds.size, False)
        frontier, (rel_row,) = O.relabel([seeds, nodes[c_row]], [nodes[c_row]])
        rel_col = np.repeat(np.arange(seeds.size, dtype=np.int64), np.diff(c_ip))
        layers.append((frontier, rel_row, rel_col, w_norm[c_perm], prob))
        # next seeds: all_indices() = distinct ids of (column ids, row ids) (src/graph.cc:757-778)
        seeds = O.unique(np.concatenate([seeds, nodes]))
    return layers


def ladies(cx, cpu_budget):
    """The layer-wise configuration: R-MAT 2.45 M / 124 M with fp32 edge weights, 2 layers of 512
    weighted picks from 512 seeds (examples/ladies/ladies_raw.py:33-54 is the harness this
    stands for), as written against Matrix and through jit.compile."""
    torch, np, gs, O, dev, args = cx.torch, cx.np, cx.gs, cx.O, cx.dev, cx.args
    from graph_sampling_amd import jit
    nodes, edges, idt = WORKLOADS[SAGE]
    idt = getattr(torch, idt)
    PICKS, B = [512, 512], 512
    indptr, indices = cx.rmat.rmat_csc(nodes, edges, seed=0, device=dev, index_dtype=idt)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    weights = 1.0 - torch.rand(edges, generator=gen, device=dev)
    A = gs.Matrix().load_csc(indptr, indices, weights)
    gen.manual_seed(4)
    steps, warm = min(args.steps, 100), min(args.warmup, 5)
    sets = [torch.randperm(nodes, generator=gen, device=dev)[:B].to(idt)
            for _ in range(warm + steps)]
    edges_of = lambda o: sum(blk.num_edges() for blk in o[1])
    ladies_sampler = make_ladies_sampler(torch)
    compiled = jit.compile(ladies_sampler, (A, sets[0], PICKS))
    out = {"workload": SAGE + " with fp32 edge weights ~U(0,1]", "batch": B,
           "picks_per_layer": PICKS, "steps": steps,
           "api": "gs.Matrix: A[:, seeds], sum(axis=1, powk=2), list_sampling_with_probs, "
                  "U[nodes, :], divide, normalize, all_indices, to_dgl_block "
                  "(examples/ladies/ladies_raw.py:8-27)"}
    first_seed = 1000
    for name, fn in (("as_written", ladies_sampler), ("compiled", compiled)):
        gs.set_seed(0)
        for s in sets[:warm]:
            fn(A, s, PICKS)
        gs.set_seed(first_seed)
        seen = []
        first = (make_ladies_sampler(torch, seen) if name == "as_written" else fn)(A, sets[warm], PICKS)
        gs.set_seed(first_seed)
        e, t = timed(torch, lambda s: edges_of(fn(A, s, PICKS)), sets[warm:])
        out[name] = {"ms_per_step": t / steps * 1e3, "value": e / t, "unit": "block edges/s"}
        if O is not None and name == "as_written":
            h_indptr = indptr.cpu().numpy()
            h_indices = indices.cpu().numpy().astype(np.int64)
            h_w = weights.cpu().numpy()
            h_seeds = sets[warm].cpu().numpy().astype(np.int64)
            # the checked run's own row probabilities decide the oracle's picks (they differ
            # from the oracle's in the last bits: float sums in another order)
            probs = [p.cpu().numpy() for p in seen]
            want = cpu_ladies(O, np, h_indptr, h_indices, h_w, h_seeds, PICKS, first_seed, probs)
            bad = []
            for l, (frontier, rel_row, rel_col, w_norm, prob) in enumerate(want):
                blk = first[1][len(PICKS) - 1 - l]
                row, col = blk.edges()
                same = {"row probabilities": np.allclose(probs[l], prob, rtol=1e-5, atol=0),
                        "frontier": np.array_equal(blk.srcdata["_ID"].cpu().numpy().astype(np.int64), frontier),
                        "rows": np.array_equal(row.cpu().numpy().astype(np.int64), rel_row),
                        "columns": np.array_equal(col.cpu().numpy().astype(np.int64), rel_col),
                        "weights": w_norm.shape == tuple(blk.edata["w"].shape) and
                        np.allclose(blk.edata["w"].cpu().numpy(), w_norm, rtol=1e-4, atol=0)}
                bad += ["layer %d %s" % (l, k) for k, v in same.items() if not v]
            if bad:
                print("bench.py: the LADIES minibatch differs from the oracle: " + ", ".join(bad),
                      file=sys.stderr)
                sys.exit(1)
            out["checked"] = ("step 0: every block's frontier and edge ends bit for bit against the "
                              "oracle (picks made by the device's row probabilities, which agree "
                              "with the oracle's at 1e-5), normalised weights at 1e-4")
            if cpu_budget > 0:
                t1 = time.perf_counter()
                done, c_edges = 0, 0
                while time.perf_counter() - t1 < cpu_budget and done < steps:
                    hs = sets[warm + done].cpu().numpy().astype(np.int64)
                    c_edges += sum(x[1].size for x in cpu_ladies(O, np, h_indptr, h_indices, h_w, hs,
                                                                 PICKS, first_seed + 2 * done))
                    done += 1
                c_s = time.perf_counter() - t1
                out["cpu_baseline"] = {
                    "value": c_edges / c_s, "unit": "block edges/s", "cores": O.num_threads(),
                    "kind": "port", "ms_per_step": c_s / done * 1e3,
                    "sample": "%d minibatches in %.1f s through the oracle's operators on host "
                              "arrays (slice, sum, A-Res pick, stable sort, slice, divide, "
                              "normalise, relabel)" % (done, c_s)}
            del h_indptr, h_indices, h_w
    del A, indptr, indices, weights
    torch.cuda.empty_cache()
    return out


def walks(cx, cpu_budget):
    """The walk configuration: 1 M uniform-random starts x 80 steps on R-MAT 4 M / 200 M, and a
    metapath walk (length 4, repeated 4 times) over three bipartite 50 M-edge relations
    (examples/randomwalk/randomwalk_fused_bench.py:65-82 is the harness this stands for)."""
    torch, np, gs, O, dev, args = cx.torch, cx.np, cx.gs, cx.O, cx.dev, cx.args
    idt = torch.int32
    W, L, REPS = 1_000_000, 80, 10
    PREFIX = 10_000
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    out = {}

    def timed_walk(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(REPS):
            tr = fn()
        torch.cuda.synchronize()
        return tr, (time.perf_counter() - t1) / REPS

    # ---- uniform walk
    N, E = 4_000_000, 200_000_000
    indptr, indices = cx.rmat.rmat_csc(N, E, seed=0, device=dev, index_dtype=idt)
    g = gs.Graph(False)
    g._CAPI_LoadCSC(indptr, indices)
    starts = torch.randint(0, N, (W,), generator=gen, device=dev).to(idt)
    gs.set_seed(50)
    first = g._CAPI_RandomWalk(starts, L)
    trace, t = timed_walk(lambda: g._CAPI_RandomWalk(starts, L))
    live = int((trace.reshape(-1)[W:] >= 0).sum())
    out["random_walk"] = {
        "workload": "rmat-4M-200M", "walkers": W, "length": L, "ms_per_call": t * 1e3,
        "live_steps": live, "value": live / t, "unit": "steps/s",
        "roofline": {"bound": "hbm", "achieved": live * 28 / t / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": live * 28 / t / 1e9 / HBM_PEAK_GBS,
                     "what": "28 B per live step (two offsets, one neighbour id, one trace entry); "
                             "each step is two dependent reads of random memory lines"},
        "api": "gs_classes.Graph._CAPI_RandomWalk"}
    if O is not None:
        h_indptr = indptr.cpu().numpy()
        h_indices = indices.cpu().numpy().astype(np.int64)
        h_starts = starts.cpu().numpy().astype(np.int64)
        # walker w's draws depend on (w, step) only: a prefix of the walkers walks the same way alone
        want = O.random_walk(h_indptr, h_indices, h_starts[:PREFIX], L, seed=50).reshape(L + 1, PREFIX)
        got = first.reshape(-1).reshape(L + 1, W)[:, :PREFIX].cpu().numpy().astype(np.int64)
        if not np.array_equal(got, want):
            print("bench.py: the random walk differs from the oracle", file=sys.stderr)
            sys.exit(1)
        out["random_walk"]["checked"] = "the first %d walkers' whole traces against the oracle" % PREFIX
        if cpu_budget > 0:
            n_cpu = W
            t1 = time.perf_counter()
            tr = O.random_walk(h_indptr, h_indices, h_starts[:n_cpu], L, seed=51)
            c_s = time.perf_counter() - t1
            c_live = int((tr[n_cpu:] >= 0).sum())
            out["random_walk"]["cpu_baseline"] = {
                "value": c_live / c_s, "unit": "steps/s", "cores": O.num_threads(), "kind": "port",
                "sample": "%d of the walkers, %d steps, in %.1f s through the C oracle" % (n_cpu, L, c_s)}
        del h_indptr, h_indices
    del g, indptr, indices, trace, first
    torch.cuda.empty_cache()

    # ---- metapath walk: user -> item -> user -> tag style relations, each R-MAT 1 M x 2 M, 50 M edges
    rel_names = ["r0", "r1", "r2"]
    rels = [cx.rmat.rmat_csc(2_000_000, 50_000_000, seed=30 + r, device=dev, index_dtype=idt,
                             num_src_nodes=2_000_000) for r in range(3)]
    mats = []
    for ip, ix in rels:
        m = gs.Matrix().load_csc(ip, ix)
        mats.append(m)
    hm = gs.HeteroMatrix()
    hm.load_from_homo(["n"], [("n", r, "n") for r in rel_names], mats)
    path = ["r0", "r1", "r2", "r1"] * 4
    mstarts = torch.randint(0, 2_000_000, (W,), generator=gen, device=dev).to(idt)
    gs.set_seed(60)
    first = hm.metapath_random_walk_fused(mstarts, path)
    trace, t = timed_walk(lambda: hm.metapath_random_walk_fused(mstarts, path))
    live = int((trace.reshape(-1)[W:] >= 0).sum())
    out["metapath_walk"] = {
        "workload": "3 relations, each rmat 2M x 2M ids / 50M edges", "walkers": W,
        "metapath": "length 4 x 4 repeats = 16 steps", "ms_per_call": t * 1e3, "live_steps": live,
        "value": live / t, "unit": "steps/s",
        "roofline": {"bound": "hbm", "achieved": live * 28 / t / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": live * 28 / t / 1e9 / HBM_PEAK_GBS,
                     "what": "28 B per live step"},
        "api": "gs_classes.HeteroGraph._CAPI_MetapathRandomWalkFused"}
    if O is not None:
        host = [(ip.cpu().numpy(), ix.cpu().numpy().astype(np.int64)) for ip, ix in rels]
        steps_rel = [rel_names.index(p) for p in path]
        h_starts = mstarts.cpu().numpy().astype(np.int64)
        want = O.metapath_walk([h[0] for h in host], [h[1] for h in host], steps_rel,
                               h_starts[:PREFIX], seed=60).reshape(len(path) + 1, PREFIX)
        got = first.reshape(-1).reshape(len(path) + 1, W)[:, :PREFIX].cpu().numpy().astype(np.int64)
        if not np.array_equal(got, want):
            print("bench.py: the metapath walk differs from the oracle", file=sys.stderr)
            sys.exit(1)
        out["metapath_walk"]["checked"] = "the first %d walkers' whole traces against the oracle" % PREFIX
        if cpu_budget > 0:
            n_cpu = W
            t1 = time.perf_counter()
            tr = O.metapath_walk([h[0] for h in host], [h[1] for h in host], steps_rel,
                                 h_starts[:n_cpu], seed=61)
            c_s = time.perf_counter() - t1
            c_live = int((tr[n_cpu:] >= 0).sum())
            out["metapath_walk"]["cpu_baseline"] = {
                "value": c_live / c_s, "unit": "steps/s", "cores": O.num_threads(), "kind": "port",
                "sample": "%d of the walkers, 16 steps, in %.1f s through the C oracle" % (n_cpu, c_s)}
    del hm, mats, rels
    torch.cuda.empty_cache()
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (one process, whole graph resident in its "
              "HBM); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    import graph_sampling_amd as gs
    from graph_sampling_amd import capi, rmat

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    timer = KernelTimer(capi.lib())  # fails loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    O = None
    if not args.no_cpu:
        from oracle import oracle as O
    cx = Ctx(torch, np, gs, capi, rmat, timer, O, dev, args)

    weighted = not args.no_weights
    legs = [x for x in args.legs.split(",") if x]
    head = graphsage(cx, args.workload, weighted, with_features=args.workload == LARGE,
                     full="headline", cpu_budget=12.0)
    out = {
        "metric": "sampled edges/sec (GSEPS), GraphSAGE [15,10,5] batch 1024, slice+sample+relabel",
        "value": head.pop("value"),
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head.pop("ms_per_step"),
        "p50_ms": head.pop("p50_ms"),
        "p90_ms": head.pop("p90_ms"),
        "latency_note": "p50/p90: one minibatch with the device drained before and after it; "
                        "ms_per_step: the timed steps back to back",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head.pop("dtype"),
        "data": "synthetic R-MAT (a=.57,b=.19,c=.19), generated on device, seed 0; edge weights "
                "1 - U[0,1) fp32, seed 1",
    }
    out.update(head)
    if not args.headline_only:
        if "config_2" in legs and args.workload != SAGE:
            out["config_2"] = leg(lambda: graphsage(cx, SAGE, False, with_features=False,
                                                    full="config2", cpu_budget=6.0))
        if "ladies" in legs:
            out["ladies"] = leg(lambda: ladies(cx, cpu_budget=6.0))
        if "walks" in legs:
            out["walks"] = leg(lambda: walks(cx, cpu_budget=1.0))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
