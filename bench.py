#!/usr/bin/env python3
"""GraphSAGE minibatch sampling benchmark (one MI355X).

One step = one [15,10,5] minibatch over 1024 fresh seed nodes on a synthetic R-MAT graph
resident in HBM: per layer a fused column slice + uniform sample without replacement, then
unique / relabel of (seeds, sampled rows); the frontier feeds the next layer.  The timed step
is ONE call of the drop-in Graph class, _CAPI_SampleLayers, which does what the loop of the
reference's examples does (examples/graphsage/batching.py:125-138) with every layer queued on
the device and the sizes collected once; the same minibatches through the per-layer calls of
that loop (_CAPI_FusedColumnwiseSlicingSampling + _CAPI_Relabel) are reported beside it
(`per_layer_api`), as are the reference's own Algorithm R, the unfused operators, the
super-batch operators, several minibatches in flight and the 111 M-node graph with u_dot_v on
every block.  Everything reaches the HIP kernels of libgs_hip.so through its C ABI.

Prints ONE JSON line: sampled edges per second, the roofline of the launch site that holds
the most GPU time (timed with hipEvents on the launch stream by the library's own hook), the
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
    ap.add_argument("--workload", default="rmat-2.45M-124M", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-steps", type=int, default=-1,
                    help="minibatches timed for the host-core baseline (-1: sized to ~15 s)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-large", action="store_true",
                    help="skip the pass over the 111 M-node / 1.6 B-edge graph")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the timed step and its roofline: for profiling the step alone")
    ap.add_argument("--api", default="layers", choices=("layers", "loop"),
                    help="what --headline-only runs: the one-call minibatch or the per-layer calls")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain device copy of the indices array (a kernel of known "
                         "traffic to scale hardware byte counters by)")
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


# ---------------------------------------------------------------------------------------
# Launch sites of one minibatch step and the bytes each launch must move at the least
# (b = bytes per id; S seeds, E sampled edges, M = S + E items, U distinct ids of a layer):
#   sample        per seed   column id b + two offsets 16 + output offset 8
#                 per edge   neighbour gather b + sampled id store b (no select_index: the
#                            graph carries no edge data, so the host layer does not ask for it)
#   insert        per item   one 8-byte slot read-modify-write 16 + slot index 4 (+ the id b when
#                            it is a launch of its own and reads the ids again)
#   compact       per item   slot index 4 + slot word 8 + first index set aside 8, per U id b
#   finish        per edge   first index 8 + prefix 8 + renamed id b; per item slot emptied 8;
#                 per seed   offsets copy 16
#   rank+rename   per item   slot index 4 + slot word 8 + distance 2, per edge renamed id b,
#                            per U id b; per item of the layer before, slot emptied 8 + index 4
#   sweep         per item   slot index 4 + slot emptied 8
def sample_bytes(b, S, E, U):
    return S * (b + 24) + E * 2 * b


def insert_bytes(b, S, E, U):
    return (S + E) * (b + 20)


def compact_bytes(b, S, E, U):
    return (S + E) * 20 + U * b


def finish_bytes(b, S, E, U):
    return E * (16 + b) + (S + E) * 8 + S * 16


def layer_sample_bytes(b, S, E, U):
    return sample_bytes(b, S, E, U) + (S + E) * 20


def layer_relabel_bytes(b, S, E, U):
    return (S + E) * 14 + E * b + U * b


def sweep_bytes(b, S, E, U):
    return (S + E) * 12


SITE_BYTES = {
    "layers": {"layer_sample": layer_sample_bytes, "layer_relabel": layer_relabel_bytes,
               "layer_sweep": sweep_bytes},
    "loop": {"sample_fused": sample_bytes, "table_insert": insert_bytes,
             "unique_compact": compact_bytes, "unique_finish": finish_bytes},
}
SITE_KERNEL = {
    "layer_sample": "sample_group_kernel<linked> (column slice + count + scan + uniform sample + "
                    "hash insert of seeds and sampled ids in one launch, all three layers)",
    "layer_relabel": "rank_linked_kernel (first-occurrence flags, their scan, frontier and renamed "
                     "ids in one launch; empties the table of the layer before)",
    "layer_sweep": "layer_sweep_kernel (empties the last layer's table slots)",
    "sample_fused": "sample_group_kernel (column slice + count + scan + uniform sample in one launch)",
    "table_insert": "table_insert_kernel (hash insert of seeds + sampled rows)",
    "unique_compact": "compact_kernel (first-occurrence flags, their scan, frontier)",
    "unique_finish": "finish_linked_kernel (renamed ids, offsets copy, table slots emptied)",
}
LAUNCHES_PER_STEP = {"layer_sweep": 1}


def step_bytes(sizes):
    """Bytes of one fused GraphSAGE minibatch by the per-unit figures of the scope table this
    build follows (reference widths: 8-byte ids): per layer 32 S + 16 E for slice + sample,
    64 (S + E) + 32 E + 16 U for unique + relabel; no table-clearing term, the table here is
    emptied slot by slot."""
    return sum(32 * S + 16 * E + 64 * (S + E) + 32 * E + 16 * U for S, E, U in sizes)


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
    read in between.  Returns (#sampled edges, per-layer (S, E, U), flat result list)."""
    parts = graph._CAPI_SampleLayers(seeds, list(FANOUTS), False)
    total, sizes, S = 0, [], seeds.numel()
    for l in range(len(FANOUTS)):
        U, E = parts[3 * l].numel(), parts[3 * l + 2].numel()
        sizes.append((S, E, U))
        total += E
        S = U
    return total, sizes, parts


def minibatch_loop(graph, seeds):
    """The same minibatch through exactly the calls of the reference's examples
    (examples/graphsage/batching.py:125-138): per layer
    _CAPI_FusedColumnwiseSlicingSampling(seeds, fanout, False) then _CAPI_Relabel()."""
    total, sizes, parts = 0, [], []
    for k in FANOUTS:
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
        frontier, num_src, num_dst, indptr, indices, e_ids, fmt = sub._CAPI_Relabel()
        E = indices.numel()
        sizes.append((num_dst, E, num_src))
        parts += [frontier, indptr, indices]
        total += E
        seeds = frontier
    return total, sizes, parts


MINIBATCH = {"layers": minibatch_layers, "loop": minibatch_loop}


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


def concurrent(torch, graph, seed_sets, workers):
    """The same minibatches with `workers` of them in flight: one host thread and one stream
    each, as a loader with sampler workers would run them.  The per-minibatch results do not
    depend on the interleaving (every thread counts its own seeds)."""
    import threading
    dev = seed_sets[0].device
    edges = [0] * workers

    def work(k):
        stream = torch.cuda.Stream(device=dev)
        with torch.cuda.stream(stream):
            for i in range(k, len(seed_sets), workers):
                torch.ops.gs_ops._CAPI_SetThreadSeed(i * len(FANOUTS))
                edges[k] += minibatch_layers(graph, seed_sets[i])[0]
            stream.synchronize()

    torch.cuda.synchronize()
    t1 = time.perf_counter()
    threads = [threading.Thread(target=work, args=(k,)) for k in range(workers)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    return sum(edges), time.perf_counter() - t1


def cpu_minibatch(O, np, indptr, indices, seeds, step):
    total = 0
    for layer, k in enumerate(FANOUTS):
        sub_indptr, _, sub_indices, _ = O.sample_uniform(indptr, indices, seeds, k, False,
                                                         seed=step * len(FANOUTS) + layer,
                                                         with_coo=False)
        frontier, _ = O.relabel([seeds, sub_indices], [sub_indices])
        total += int(sub_indptr[-1])
        seeds = frontier
    return total, seeds


def columns_of(torch, indptr, indices, cols):
    """(offsets, neighbour ids) of the columns `cols`, cut out of the graph with plain torch
    indexing (no library kernel): what the checker below hands to the oracle."""
    starts = indptr[cols]
    deg = indptr[cols + 1] - starts
    offsets = torch.zeros(cols.numel() + 1, dtype=torch.int64, device=indptr.device)
    torch.cumsum(deg, 0, out=offsets[1:])
    total = int(offsets[-1])
    owner = torch.repeat_interleave(torch.arange(cols.numel(), device=indptr.device), deg,
                                    output_size=total)
    pos = torch.arange(total, device=indptr.device) - offsets[owner] + starts[owner]
    return offsets, indices[pos]


def check_against_oracle(torch, np, O, indptr, indices, seeds, first_seed, parts):
    """The checker: the minibatch `parts` ([frontier, offsets, renamed ids] per layer) against
    the oracle run layer by layer with the same draws.  The oracle gets each layer's columns
    as a small graph of their own (the draws of a column depend on its place in the call, not
    on its id), so a graph of any size is checked without a host copy of it."""
    cols = seeds.long()
    for l, k in enumerate(FANOUTS):
        sub_ptr, sub_idx = columns_of(torch, indptr, indices, cols)
        h_ptr, h_idx = sub_ptr.cpu().numpy(), sub_idx.cpu().numpy().astype(np.int64)
        h_cols = cols.cpu().numpy()
        w_ptr, _, w_rows, _ = O.sample_uniform(h_ptr, h_idx, np.arange(h_cols.size, dtype=np.int64),
                                               k, False, seed=first_seed + l, with_coo=False)
        w_frontier, (w_renamed,) = O.relabel([h_cols, w_rows], [w_rows])
        got = [p.cpu().numpy().astype(np.int64) for p in parts[3 * l:3 * l + 3]]
        if not (np.array_equal(got[0], w_frontier) and np.array_equal(got[1], w_ptr)
                and np.array_equal(got[2], w_renamed)):
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
    achieved = sample_bytes(b, S, E, 0) / t / 1e9
    return {"kernel": "sample_row_lane_kernel (the one-launch sampler from 2^18 columns on: one row "
                      "per lane, edge-parallel fill)", "seeds": S, "fanout": 10, "sampled_edges": E,
            "launch_us": t * 1e6, "achieved": achieved, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS}


def timed(torch, fn, sets):
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    edges = 0
    for s in sets:
        edges += fn(s)
    torch.cuda.synchronize()
    return edges, time.perf_counter() - t1


def large_graph(torch, np, gs, capi, rmat, timer, args, dev, O):
    """Configuration 5: the timed step on R-MAT 111 M nodes / 1.6 B edges, then u_dot_v with
    64-d fp32 node features on every block (lhs = the block's source features, gathered by
    the frontier; rhs = its destination features, which are the first rows of the same
    gather).  Step 0 is compared with the oracle (ids bit for bit, dot products at 1e-5)."""
    nodes, edges, idt = WORKLOADS[LARGE]
    idt = getattr(torch, idt)
    t0 = time.perf_counter()
    indptr, indices = rmat.rmat_csc(nodes, edges, seed=0, device=dev, index_dtype=idt)
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    features = torch.rand(nodes, FEATURE_DIM, generator=gen, device=dev) - 0.5
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    graph = gs.Graph(False)
    graph._CAPI_LoadCSC(indptr, indices)
    gen.manual_seed(2)
    sets = [torch.randperm(nodes, generator=gen, device=dev)[:BATCH].to(idt)
            for _ in range(args.warmup + args.steps)]

    def dots(parts):
        outs = []
        for l in range(len(FANOUTS)):
            frontier, offsets, renamed = parts[3 * l:3 * l + 3]
            h = features.index_select(0, frontier)  # source features; seeds come first
            out = torch.empty(renamed.numel(), 1, device=dev)
            capi.sddmm_csc("dot", offsets, renamed, None, None, h, h[:offsets.numel() - 1], out,
                           0, 2, FEATURE_DIM, FEATURE_DIM, 1, FEATURE_DIM)
            outs.append(out)
        return outs

    def step(seeds):
        n, sizes, parts = minibatch_layers(graph, seeds)
        dots(parts)
        return n

    def sample_only(seeds):
        return minibatch_layers(graph, seeds)[0]

    torch.ops.gs_ops._CAPI_SetSeed(0)
    for s in sets[:args.warmup]:
        step(s)
    # the checker, untimed: step 0 of the timed region
    first_seed = args.warmup * len(FANOUTS)
    torch.ops.gs_ops._CAPI_SetSeed(first_seed)
    n0, sizes0, parts0 = minibatch_layers(graph, sets[args.warmup])
    checked = None
    if O is not None:
        ok = check_against_oracle(torch, np, O, indptr, indices, sets[args.warmup], first_seed, parts0)
        for l, out in enumerate(dots(parts0)):
            frontier, offsets, renamed = parts0[3 * l:3 * l + 3]
            h = features[frontier.long()]
            col = torch.repeat_interleave(torch.arange(offsets.numel() - 1, device=dev),
                                          offsets[1:] - offsets[:-1])
            want = (h[renamed.long()] * h[col]).sum(-1, keepdim=True)
            ok = ok and bool(torch.allclose(out, want, rtol=1e-5, atol=1e-6))
        if not ok:
            print("bench.py: the minibatch on %s differs from the oracle" % LARGE, file=sys.stderr)
            sys.exit(1)
        checked = "step 0: ids bit for bit against the oracle, u_dot_v at 1e-5 against a torch gather-and-dot"
    torch.ops.gs_ops._CAPI_SetSeed(first_seed)
    e_all, s_all = timed(torch, step, sets[args.warmup:])
    torch.ops.gs_ops._CAPI_SetSeed(first_seed)
    e_smp, s_smp = timed(torch, sample_only, sets[args.warmup:])
    timer.enable("sddmm_dot")
    for s in sets[args.warmup:args.warmup + 20]:
        step(s)
    torch.cuda.synchronize()
    d_ms, d_n, _ = timer.collect()
    timer.enable("")
    # dot of two 64-float rows per edge: 2 x 256 B of features + 12 B of ids + 4 B out
    dot_bytes = sum(E for _, E, _ in sizes0) / len(FANOUTS) * (2 * 4 * FEATURE_DIM + 12 + 4)
    dot_gbs = dot_bytes / (d_ms * 1e-3 / d_n) / 1e9 if d_n else None
    out = {"workload": LARGE, "nodes": nodes, "edges": edges, "feature_dim": FEATURE_DIM,
           "graph_build_s": round(build_s, 2), "steps": args.steps,
           "ms_per_step": s_all / args.steps * 1e3, "value": e_all / s_all,
           "sampling_only": {"ms_per_step": s_smp / args.steps * 1e3, "value": e_smp / s_smp},
           "step0_layers_S_E_U": sizes0, "checked": checked,
           "sddmm_dot": {"avg_launch_us": d_ms * 1e3 / d_n if d_n else None, "achieved": dot_gbs,
                         "unit": "GB/s", "frac": dot_gbs / HBM_PEAK_GBS if dot_gbs else None,
                         "what": "u_dot_v launches of the three blocks (2.4 k to 125 k edges each)"},
           "what": "the timed step (one _CAPI_SampleLayers call) on configuration 5's graph, then "
                   "features[frontier] and gs_sddmm_csc(dot) on each of the three blocks"}
    del graph, indptr, indices, features
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
    nodes, edges, idt = WORKLOADS[args.workload]
    idt = getattr(torch, idt)
    b = 4 if idt == torch.int32 else 8
    api = args.api if args.headline_only else "layers"
    step_fn = MINIBATCH[api]
    O = None
    if not args.no_cpu:
        from oracle import oracle as O

    t0 = time.perf_counter()
    indptr, indices = rmat.rmat_csc(nodes, edges, seed=0, device=dev, index_dtype=idt)
    torch.cuda.synchronize()
    gen_s = time.perf_counter() - t0

    graph = gs.Graph(False)
    graph._CAPI_LoadCSC(indptr, indices)
    if args.calibration_copy:
        torch.empty_like(indices).copy_(indices)
        torch.cuda.synchronize()

    gen = torch.Generator(device=dev)
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
    layer_sizes = None
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
            algo_bytes += SITE_BYTES[api][dominant](b, *sizes[-1])
        else:
            algo_bytes += sum(SITE_BYTES[api][dominant](b, *z) for z in sizes)
        whole_step_bytes += step_bytes(sizes)

    # the checker: step 0 of the timed region must agree with the oracle bit for bit
    if O is not None and not check_against_oracle(torch, np, O, indptr, indices, timed_sets[0],
                                                  first_seed, first[1]):
        print("bench.py: GPU minibatch differs from the oracle on the same seeds and draws",
              file=sys.stderr)
        sys.exit(1)

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

    extras = not args.headline_only
    ops = torch.ops.gs_ops

    # the per-layer calls of the reference's loop on the same seed sets and draws
    per_layer = None
    if extras:
        torch.ops.gs_ops._CAPI_SetSeed(0)
        for s in seed_sets[:args.warmup]:
            minibatch_loop(graph, s)
        pl_e, pl_s = timed(torch, lambda s: minibatch_loop(graph, s)[0], timed_sets)
        torch.ops.gs_ops._CAPI_SetSeed(first_seed)
        same = all(torch.equal(x, y) for x, y in zip(minibatch_loop(graph, timed_sets[0])[2], first[1]))
        per_layer = {"ms_per_step": pl_s / args.steps * 1e3, "value": pl_e / pl_s,
                     "identical_to_headline_step0": bool(same),
                     "what": "_CAPI_FusedColumnwiseSlicingSampling + _CAPI_Relabel per layer "
                             "(examples/graphsage/batching.py:125-138): one host wait per layer"}

    # the reference's own selection algorithm (Algorithm R, src/cuda/sampling.cu:70-92) on
    # the same seed sets: the count / reservoir / gather kernels instead of the one-launch sampler
    reservoir = None
    if extras:
        ops._CAPI_SetSampleAlgo(1)
        rs_steps = min(args.steps, 50)
        for s in seed_sets[:3]:
            minibatch_loop(graph, s)
        rs_e, rs_s = timed(torch, lambda s: minibatch_loop(graph, s)[0], timed_sets[:rs_steps])
        ops._CAPI_SetSampleAlgo(0)
        reservoir = {"ms_per_step": rs_s / rs_steps * 1e3, "value": rs_e / rs_s, "steps": rs_steps,
                     "what": "GS_SAMPLE_RESERVOIR through the per-layer calls: deg - fanout draws per "
                             "column, output in slot order, bit-exact against the reference's "
                             "draw sequence under replay"}

    # the unfused operator sequence on the same seed sets
    nf = None
    if extras:
        nf_steps = min(args.steps, 50)
        for s in seed_sets[:3]:
            minibatch_nonfused(graph, s)
        nf_e, nf_s = timed(torch, lambda s: minibatch_nonfused(graph, s), timed_sets[:nf_steps])
        nf = {"ms_per_step": nf_s / nf_steps * 1e3, "value": nf_e / nf_s, "steps": nf_steps,
              "what": "Slicing -> Sampling -> Relabel per layer instead of the fused sampler"}

    # SUPER minibatches per call through the batch operators, on seed sets of its own
    sb = None
    if extras:
        groups = [[fresh_seeds() for _ in range(SUPER)] for _ in range(3)]
        super_batch(torch, graph, groups[0])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        sb_edges = 0
        sb_sizes = None
        for grp in groups:
            n, sb_sizes, _ = super_batch(torch, graph, grp)
            sb_edges += n
        torch.cuda.synchronize()
        sb_s = time.perf_counter() - t1
        sb_sites = {}
        for site in ("sample_fused", "batch_init", "batch_insert", "batch_compact", "batch_finish"):
            timer.enable(site)
            super_batch(torch, graph, groups[0])
            torch.cuda.synchronize()
            ms, n, per = timer.collect()
            sb_sites[site] = (ms, per)
        timer.enable("")
        sb_dom = max(sb_sites, key=lambda k: sb_sites[k][0])
        # the dominant site's largest launch (the third layer) against its bytes
        S3, E3, U3 = sb_sizes[-1]
        M3 = S3 + E3
        sb_bytes = {"sample_fused": sample_bytes(b, S3, E3, U3),
                    "batch_init": 4 * M3 * 8,                 # one 8-byte slot per table entry, 4 per item
                    "batch_insert": M3 * (b + 16 + 4 + 8),     # id, slot RMW, slot index, batch offsets
                    "batch_compact": M3 * 20 + U3 * b,
                    "batch_finish": E3 * (16 + b) + M3 * 4}[sb_dom]
        t3 = sb_sites[sb_dom][1][-1] * 1e-3
        sb = {"minibatches_per_call": SUPER, "calls": len(groups),
              "ms_per_minibatch": sb_s / (len(groups) * SUPER) * 1e3, "value": sb_edges / sb_s,
              "layers_S_E_U": sb_sizes,
              "roofline": {"bound": "hbm", "kernel": sb_dom + " (third layer's launch)",
                           "achieved": sb_bytes / t3 / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": sb_bytes / t3 / 1e9 / HBM_PEAK_GBS, "launch_us": t3 * 1e6,
                           "algorithmic_bytes": sb_bytes,
                           "gpu_ms_by_site": {k: round(v[0], 4) for k, v in sb_sites.items()}},
              "what": "fused sampling + GetBatchCSC + BatchCSRRelabel + splits over 64 minibatches "
                      "of 1024 seeds at once; every minibatch is relabelled on its own"}
        del groups

    # the same minibatches, four in flight
    WORKERS = 4
    cc = None
    if extras:
        concurrent(torch, graph, seed_sets[:4 * WORKERS], WORKERS)
        cc_edges, cc_s = concurrent(torch, graph, timed_sets, WORKERS)
        cc = {"workers": WORKERS, "ms_per_step": cc_s / args.steps * 1e3,
              "value": cc_edges / cc_s,
              "what": "the timed minibatches again with four in flight, one host thread and one "
                      "stream each"}

    # the same minibatches with 64-bit ids, the reference's only id type
    wide = None
    if extras and idt == torch.int32 and edges <= 200_000_000:
        graph64 = gs.Graph(False)
        graph64._CAPI_LoadCSC(indptr, indices.long())
        sets64 = [s.long() for s in seed_sets]
        for s in sets64[:args.warmup]:
            minibatch_layers(graph64, s)
        w_e, w_s = timed(torch, lambda s: minibatch_layers(graph64, s)[0], sets64[args.warmup:])
        wide = {"ms_per_step": w_s / args.steps * 1e3, "value": w_e / w_s,
                "what": "the timed minibatches on the same graph with int64 ids"}
        del graph64, sets64

    # the same again by the C++ layer's own pool of sampler threads (no interpreter in the
    # loop), 32 minibatches per call as a loader with that prefetch depth would ask for them
    pool = None
    if extras:
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
        pool = {"workers": POOL, "minibatches_per_call": DEPTH,
                "ms_per_step": pool_s / len(timed_sets) * 1e3, "value": pool_edges / pool_s,
                "what": "the timed minibatches through gs_ops._CAPI_SampleBlocks: three host threads "
                        "of the C++ layer, one stream each, every minibatch queued whole"}

    out = {
        "metric": "sampled edges/sec (GSEPS), GraphSAGE [15,10,5] batch 1024, slice+sample+relabel",
        "value": sampled / elapsed,
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "p50_ms": p50,
        "p90_ms": p90,
        "latency_note": "p50/p90: one minibatch with the device drained before and after it; "
                        "ms_per_step: the timed steps back to back",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int32" if idt == torch.int32 else "int64",
        "data": "synthetic R-MAT (a=.57,b=.19,c=.19), generated on device, seed 0",
        "config": {"workload": args.workload, "nodes": nodes, "edges": edges, "batch": BATCH,
                   "fanouts": list(FANOUTS), "last_step_layers_S_E_U": layer_sizes,
                   "graph_build_s": round(gen_s, 2),
                   "api": "gs_classes.Graph._CAPI_SampleLayers (one call per minibatch)"
                          if api == "layers" else
                          "gs_classes.Graph._CAPI_FusedColumnwiseSlicingSampling + _CAPI_Relabel per layer"},
        "per_layer_api": per_layer,
        "reservoir_mode": reservoir,
        "unfused_path": nf,
        "super_batch": sb,
        "concurrent": cc,
        "sampler_pool": pool,
        "int64_ids": wide,
        "large_graph": None,
        "roofline": None,
        "step_roofline": None,
        "cpu_baseline": None,
    }
    step_gbs = whole_step_bytes / elapsed / 1e9
    out["step_roofline"] = {
        "bound": "hbm", "achieved": step_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": step_gbs / HBM_PEAK_GBS, "bytes_per_step": whole_step_bytes / args.steps,
        "what": "per layer 32 S + 16 E (slice + sample) + 64 (S + E) + 32 E + 16 U (unique + "
                "relabel), reference id widths, over ms_per_step"}
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
            "traffic": traffic_from_profile(dominant, args.workload),
            "traffic_source": "profiles/%s_%s_hbm_counters.txt" % (dominant, args.workload),
            "launches": per_step * args.steps,
            "launches_timed": k_launches,
            "avg_launch_us": avg_s * 1e6,
            "empty_event_pair_us": empty_pair_us(torch),
            "algorithmic_bytes_per_launch": bytes_per_launch,
            "gpu_ms_per_step_by_site": {k: round(v, 4) for k, v in site_ms.items()},
        }
        out["roofline_saturated"] = saturated(torch, graph, timer, nodes, idt, dev, b)

    if O is not None:
        h_indptr = indptr.cpu().numpy()
        h_indices = indices.cpu().numpy().astype(np.int64)
        h_seeds = [s.cpu().numpy().astype(np.int64) for s in timed_sets]
        n_ref, f_ref = cpu_minibatch(O, np, h_indptr, h_indices, h_seeds[0], args.warmup)
        if n_ref != first[0] or not np.array_equal(f_ref, first[1][-3].cpu().numpy()):
            print("bench.py: GPU minibatch differs from the oracle on the same seeds and draws",
                  file=sys.stderr)
            sys.exit(1)
        t1 = time.perf_counter()
        done = 0
        cpu_edges = 0
        budget = 15.0
        # ten passes over the timed seed sets (fresh draws every pass), at most `budget` seconds
        limit = args.cpu_steps if args.cpu_steps > 0 else 10 * len(h_seeds)
        while done < limit and (args.cpu_steps > 0 or time.perf_counter() - t1 < budget):
            cpu_edges += cpu_minibatch(O, np, h_indptr, h_indices, h_seeds[done % len(h_seeds)],
                                       args.warmup + done)[0]
            done += 1
        cpu_s = time.perf_counter() - t1
        out["cpu_baseline"] = {
            "value": cpu_edges / cpu_s,
            "unit": "edges/s",
            "cores": O.num_threads(),
            "kind": "port",
            "sample": "%d minibatches in %.1f s: the timed seed sets (same seeds; the first pass "
                      "with the same draws) through the C oracle, OpenMP over rows; unique is "
                      "single-threaded; step 0 compared with the GPU result bit for bit"
                      % (done, cpu_s),
            "ms_per_step": cpu_s / done * 1e3,
        }
        del h_indptr, h_indices

    if extras and not args.no_large and args.workload != LARGE:
        del graph, indptr, indices
        torch.cuda.empty_cache()
        out["large_graph"] = large_graph(torch, np, gs, capi, rmat, timer, args, dev, O)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
