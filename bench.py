#!/usr/bin/env python3
"""GraphSAGE minibatch sampling benchmark (one MI355X).

One step = one [15,10,5] minibatch over 1024 fresh seed nodes on a synthetic
R-MAT graph: per layer a fused column slice + uniform sample without
replacement, then unique/relabel of (seeds, sampled rows); the frontier feeds
the next layer.  The step is written against the drop-in Graph class (the
reference's _CAPI_* method names), which calls the HIP kernels of libgs_hip.so
through its C ABI; the graph is resident in HBM.  Prints ONE JSON line (sampled
edges per second) carrying the roofline of the dominant kernel (timed with
hipEvents on the launch stream by the library's own hook) and a host-core
baseline of the same minibatches.
"""
import argparse
import ctypes
import json
import os
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
FANOUTS = (15, 10, 5)
BATCH = 1024
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the roofline kernel on the default workload, read from hardware
# counters (2.0 x FETCH_SIZE + 1.0 x WRITE_SIZE; the factors come from a device copy of
# known size): profiles/sample_fused_rmat-2.45M-124M_hbm_counters.txt.  The counters cannot
# be read from inside this process, so the figure is carried here.
TRAFFIC_BYTES_PER_LAUNCH = {("rmat-2.45M-124M", "sample_fused"): 11629119}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="rmat-2.45M-124M", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-steps", type=int, default=-1,
                    help="minibatches timed for the host-core baseline (-1: sized to ~15 s)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the passes reported beside the headline (unfused operators, "
                         "super-batch, four in flight): for profiling the timed step alone")
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


# launch sites of one minibatch step and the bytes each launch must move at the
# least (id_bytes b; S seeds, E sampled edges, M = S + E items, U unique ids):
#   sample_fused  : per seed  column id b + two offsets 16 + output offset 8,
#                   per edge  neighbour gather b + sub_indices b (no select_index: the graph
#                   carries no edge data, so the host layer does not ask for it)
#   table_insert  : per item  id b + one 8-byte slot read-modify-write 16 + slot index 4
#   unique_finish : per item  slot index 4 + slot 8 + rank 8, relabeled id b, frontier b per U
SITES = ("sample_fused", "table_init", "table_insert", "unique_compact", "unique_finish")
# (unique_finish is the relabel lookup kernel)


def floyd_bytes(b, S, E):
    return S * (b + 24) + E * 2 * b


def insert_bytes(b, S, E):
    return (S + E) * (b + 20)


SITE_BYTES = {"sample_fused": floyd_bytes, "table_insert": insert_bytes}
SITE_KERNEL = {
    "sample_fused": "sample_fused_kernel (column slice + count + scan + uniform sample in one "
                    "launch, all three layers)",
    "table_insert": "table_insert_kernel (hash insert of seeds + sampled rows, all three layers)",
}


def minibatch(graph, seeds):
    """One GraphSAGE minibatch through the drop-in Graph API, exactly the calls of the
    reference's examples (examples/graphsage/batching.py:125-138): per layer
    _CAPI_FusedColumnwiseSlicingSampling(seeds, fanout, False) then _CAPI_Relabel().
    Returns (#sampled edges, per-layer (S, E, U), final frontier)."""
    total = 0
    sizes = []
    for k in FANOUTS:
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
        frontier, num_src, num_dst, indptr, indices, e_ids, fmt = sub._CAPI_Relabel()
        E = indices.numel()
        sizes.append((num_dst, E, num_src))
        total += E
        seeds = frontier
    return total, sizes, seeds


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
    into per-minibatch blocks."""
    seeds = torch.cat(seed_sets)
    ptr = torch.arange(len(seed_sets) + 1, dtype=torch.int64, device=seeds.device) * BATCH
    total = 0
    ops = torch.ops.gs_ops
    for k in FANOUTS:
        sub = graph._CAPI_FusedColumnwiseSlicingSampling(seeds, k, False)
        indptr, indices, indices_ptr = sub._CAPI_GetBatchCSC(ptr)
        uni, uni_ptr, rel, indices_ptr = ops.BatchCSRRelabel(seeds, ptr, indices, indices_ptr)
        blocks = (ops.SplitByOffset(uni, uni_ptr), ops.IndptrSplitByOffset(indptr, ptr),
                  ops.SplitByOffset(rel, indices_ptr))
        total += indices.numel()
        seeds, ptr = uni, uni_ptr
    return total, blocks


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
                edges[k] += minibatch(graph, seed_sets[i])[0]
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


def saturated(torch, graph, timer, nodes, idt, dev, b):
    """The same sampler launch at a size that fills the chip (4M seed columns drawn with
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
    achieved = floyd_bytes(b, S, E) / t / 1e9
    return {"seeds": S, "fanout": 10, "sampled_edges": E, "launch_us": t * 1e6,
            "achieved": achieved, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS}


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
    torch.cuda.synchronize()

    # the Graph API draws seed, seed+1, ... per sampling call: 3 calls per step
    torch.ops.gs_ops._CAPI_SetSeed(0)
    for i in range(args.warmup):
        minibatch(graph, seed_sets[i])
    torch.cuda.synchronize()

    # which launch site holds the most GPU time: one untimed step per site
    site_ms = {}
    probe = seed_sets[0]
    for site in SITES:
        timer.enable(site)
        minibatch(graph, probe)
        torch.cuda.synchronize()
        site_ms[site] = timer.collect()[0]
    dominant = max(SITE_BYTES, key=lambda k: site_ms[k])

    torch.ops.gs_ops._CAPI_SetSeed(args.warmup * len(FANOUTS))
    # every 4th launch of the dominant site is bracketed by an event pair: with three
    # launches per step that visits the three layers in turn, and keeps the pairs' own
    # queue time (about 6 us each, as long as the kernel) mostly out of the measurement
    timer.enable(dominant, every=4)
    sampled = 0
    layer_sizes = None
    first = None
    algo_bytes = 0
    b = 4 if idt == torch.int32 else 8
    torch.cuda.synchronize()
    t_begin = time.perf_counter()
    for i in range(args.steps):
        # a step ends when the host holds every tensor size of the minibatch (the last
        # relabel hands back the frontier length); nothing else synchronises inside the loop
        n, sizes, frontier = minibatch(graph, seed_sets[args.warmup + i])
        sampled += n
        layer_sizes = sizes
        algo_bytes += sum(SITE_BYTES[dominant](b, S, E) for S, E, _ in sizes)
        if first is None:
            first = (n, frontier)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_begin
    k_ms, k_launches, _ = timer.collect()
    timer.enable("")

    # latency of one minibatch with the device drained before and after it (untimed pass over
    # the same seed sets)
    lat = []
    for i in range(args.steps):
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        minibatch(graph, seed_sets[args.warmup + i])
        torch.cuda.synchronize()
        lat.append(time.perf_counter() - t1)
    lat.sort()
    p50 = lat[len(lat) // 2] * 1e3
    p90 = lat[min(len(lat) - 1, int(len(lat) * 0.9))] * 1e3

    # the unfused operator sequence on the same seed sets (reported beside the headline)
    extras = not args.headline_only
    nf = None
    if extras:
        nf_steps = min(args.steps, 50)
        for i in range(3):
            minibatch_nonfused(graph, seed_sets[i])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        nf_edges = 0
        for i in range(nf_steps):
            nf_edges += minibatch_nonfused(graph, seed_sets[args.warmup + i])
        torch.cuda.synchronize()
        nf_s = time.perf_counter() - t1
        nf = {"ms_per_step": nf_s / nf_steps * 1e3, "value": nf_edges / nf_s, "steps": nf_steps,
              "what": "Slicing -> Sampling -> Relabel per layer instead of the fused sampler"}

    # the same minibatches, SUPER of them per call (reported beside the headline)
    SUPER = 64
    groups = [seed_sets[i:i + SUPER] for i in range(0, len(seed_sets) - SUPER + 1, SUPER)][:8]
    sb = None
    if groups and extras:
        super_batch(torch, graph, groups[0])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        sb_edges = 0
        for grp in groups:
            sb_edges += super_batch(torch, graph, grp)[0]
        torch.cuda.synchronize()
        sb_s = time.perf_counter() - t1
        sb = {"minibatches_per_call": SUPER, "calls": len(groups),
              "ms_per_minibatch": sb_s / (len(groups) * SUPER) * 1e3, "value": sb_edges / sb_s,
              "what": "fused sampling + GetBatchCSC + BatchCSRRelabel + splits over 64 minibatches "
                      "of 1024 seeds at once; every minibatch is relabelled on its own"}

    # the same minibatches, four in flight (reported beside the headline)
    WORKERS = 4
    cc = None
    if extras:
        concurrent(torch, graph, seed_sets[:4 * WORKERS], WORKERS)
        cc_edges, cc_s = concurrent(torch, graph, seed_sets[args.warmup:], WORKERS)
        cc = {"workers": WORKERS, "ms_per_step": cc_s / args.steps * 1e3,
              "value": cc_edges / cc_s,
              "what": "the timed minibatches again with four in flight, one host thread and one "
                      "stream each"}

    # the same minibatches with 64-bit ids, the reference's only id type (beside the headline)
    wide = None
    if extras and idt == torch.int32 and edges <= 200_000_000:
        graph64 = gs.Graph(False)
        graph64._CAPI_LoadCSC(indptr, indices.long())
        sets64 = [s.long() for s in seed_sets]
        for i in range(args.warmup):
            minibatch(graph64, sets64[i])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        wide_edges = 0
        for i in range(args.steps):
            wide_edges += minibatch(graph64, sets64[args.warmup + i])[0]
        torch.cuda.synchronize()
        wide_s = time.perf_counter() - t1
        wide = {"ms_per_step": wide_s / args.steps * 1e3, "value": wide_edges / wide_s,
                "what": "the timed minibatches on the same graph with int64 ids"}
        del graph64, sets64

    # the same again by the C++ layer's own pool of sampler threads (no interpreter in the
    # loop), 32 minibatches per call as a loader with that prefetch depth would ask for them
    pool = None
    if extras:
        ops = torch.ops.gs_ops
        DEPTH = 32
        timed_sets = seed_sets[args.warmup:]
        ops._CAPI_SampleBlocks(graph, seed_sets[:DEPTH], FANOUTS, False, WORKERS, 0)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        pool_edges = 0
        for c0 in range(0, len(timed_sets), DEPTH):
            res = ops._CAPI_SampleBlocks(graph, timed_sets[c0:c0 + DEPTH], FANOUTS, False, WORKERS,
                                         c0 * len(FANOUTS))
            pool_edges += sum(int(parts[3 * l + 2].numel()) for parts in res
                              for l in range(len(FANOUTS)))
            del res
        torch.cuda.synchronize()
        pool_s = time.perf_counter() - t1
        pool = {"workers": WORKERS, "minibatches_per_call": DEPTH,
                "ms_per_step": pool_s / len(timed_sets) * 1e3, "value": pool_edges / pool_s,
                "what": "the timed minibatches through gs_ops._CAPI_SampleBlocks: four host threads "
                        "of the C++ layer, one stream each"}

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
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int32" if idt == torch.int32 else "int64",
        "data": "synthetic R-MAT (a=.57,b=.19,c=.19), generated on device, seed 0",
        "config": {"workload": args.workload, "nodes": nodes, "edges": edges, "batch": BATCH,
                   "fanouts": list(FANOUTS), "last_step_layers_S_E_U": layer_sizes,
                   "graph_build_s": round(gen_s, 2)},
        "unfused_path": nf,
        "super_batch": sb,
        "concurrent": cc,
        "sampler_pool": pool,
        "int64_ids": wide,
        "roofline": None,
        "cpu_baseline": None,
    }
    if k_launches:
        avg_s = k_ms * 1e-3 / k_launches
        bytes_per_launch = algo_bytes / (len(FANOUTS) * args.steps)
        achieved = bytes_per_launch / avg_s / 1e9
        out["roofline"] = {
            "bound": "hbm",
            "kernel": SITE_KERNEL[dominant],
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": TRAFFIC_BYTES_PER_LAUNCH.get((args.workload, dominant)),
            "launches": len(FANOUTS) * args.steps,
            "launches_timed": k_launches,
            "avg_launch_us": avg_s * 1e6,
            "algorithmic_bytes_per_launch": bytes_per_launch,
            "share_of_gpu_time_by_site_ms": {k: round(v, 4) for k, v in site_ms.items()},
        }
        out["roofline_saturated"] = saturated(torch, graph, timer, nodes, idt, dev, b)

    if not args.no_cpu:
        from oracle import oracle as O
        h_indptr = indptr.cpu().numpy()
        h_indices = indices.cpu().numpy().astype(np.int64)
        h_seeds = [s.cpu().numpy().astype(np.int64) for s in seed_sets[args.warmup:]]
        # the checker: step 0 of the timed region must agree with the oracle bit for bit
        n_ref, f_ref = cpu_minibatch(O, np, h_indptr, h_indices, h_seeds[0], args.warmup)
        if n_ref != first[0] or not np.array_equal(f_ref, first[1].cpu().numpy()):
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
    print(json.dumps(out))


if __name__ == "__main__":
    main()
