#!/usr/bin/env python3
"""GraphSAGE minibatch sampling benchmark (one MI355X).

One step = one [15,10,5] minibatch over 1024 fresh seed nodes on a synthetic
R-MAT graph: per layer a fused column slice + uniform sample without
replacement, then unique/relabel of (seeds, sampled rows); the frontier feeds
the next layer.  Everything runs through the C ABI of libgs_hip.so with the
graph resident in HBM.  Prints ONE JSON line (sampled edges per second).
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


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="rmat-2.45M-124M", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-steps", type=int, default=-1,
                    help="minibatches timed for the host-core baseline (-1: sized to ~15 s)")
    ap.add_argument("--no-cpu", action="store_true")
    return ap.parse_args()


class HipEvents:
    """hipEvent pairs on the stream the kernels run on (torch's current stream)."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")

    def create(self):
        ev = ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(ev)) == 0
        return ev

    def record(self, ev, stream):
        assert self.hip.hipEventRecord(ev, ctypes.c_void_p(stream)) == 0

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        assert self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value


def minibatch(capi, torch, indptr, indices, seeds, step_seed):
    """One GraphSAGE minibatch.  Returns (#sampled edges, per-layer sizes, final frontier)."""
    total = 0
    sizes = []
    for layer, k in enumerate(FANOUTS):
        sub_indptr, sub_indices, select_index, _ = capi.sample_uniform(
            indptr, indices, seeds, k, False, seed=step_seed * 16 + layer)
        E = int(sub_indptr[-1].item())
        rows = sub_indices[:E]
        frontier, num, outs = capi.unique_relabel([seeds, rows], [rows])
        U = int(num.item())
        sizes.append((seeds.numel(), E, U))
        total += E
        seeds = frontier[:U]
    return total, sizes, seeds


def cpu_minibatch(O, np, indptr, indices, seeds, step_seed):
    total = 0
    for layer, k in enumerate(FANOUTS):
        sub_indptr, _, sub_indices, _ = O.sample_uniform(indptr, indices, seeds, k, False,
                                                         seed=step_seed * 16 + layer, with_coo=False)
        frontier, _ = O.relabel([seeds, sub_indices], [sub_indices])
        total += int(sub_indptr[-1])
        seeds = frontier
    return total


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (one process, whole graph resident in its "
              "HBM); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    from graph_sampling_amd import capi, rmat

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    capi.lib()  # fail loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    nodes, edges, idt = WORKLOADS[args.workload]
    idt = getattr(torch, idt)

    t0 = time.perf_counter()
    indptr, indices = rmat.rmat_csc(nodes, edges, seed=0, device=dev, index_dtype=idt)
    torch.cuda.synchronize()
    gen_s = time.perf_counter() - t0

    gen = torch.Generator(device=dev)
    gen.manual_seed(2)

    def fresh_seeds():
        return torch.randperm(nodes, generator=gen, device=dev)[:BATCH].to(idt)

    seed_sets = [fresh_seeds() for _ in range(args.warmup + args.steps)]
    torch.cuda.synchronize()

    for i in range(args.warmup):
        minibatch(capi, torch, indptr, indices, seed_sets[i], i)
    torch.cuda.synchronize()

    lat = []
    sampled = 0
    layer_sizes = None
    t_begin = time.perf_counter()
    for i in range(args.steps):
        t1 = time.perf_counter()
        n, sizes, _ = minibatch(capi, torch, indptr, indices, seed_sets[args.warmup + i],
                                args.warmup + i)
        torch.cuda.synchronize()
        lat.append(time.perf_counter() - t1)
        sampled += n
        layer_sizes = sizes
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_begin
    lat.sort()
    p50 = lat[len(lat) // 2] * 1e3
    p90 = lat[min(len(lat) - 1, int(len(lat) * 0.9))] * 1e3

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
        "roofline": None,
        "cpu_baseline": None,
    }

    if not args.no_cpu:
        from oracle import oracle as O
        h_indptr = indptr.cpu().numpy()
        h_indices = indices.cpu().numpy().astype(np.int64)
        h_seeds = [s.cpu().numpy().astype(np.int64) for s in seed_sets[args.warmup:]]
        cpu_minibatch(O, np, h_indptr, h_indices, h_seeds[0], args.warmup)  # warm
        t1 = time.perf_counter()
        done = 0
        cpu_edges = 0
        budget = 15.0
        limit = args.cpu_steps if args.cpu_steps > 0 else len(h_seeds)
        while done < limit and (args.cpu_steps > 0 or time.perf_counter() - t1 < budget):
            cpu_edges += cpu_minibatch(O, np, h_indptr, h_indices, h_seeds[done], args.warmup + done)
            done += 1
        cpu_s = time.perf_counter() - t1
        out["cpu_baseline"] = {
            "value": cpu_edges / cpu_s,
            "unit": "edges/s",
            "cores": O.num_threads(),
            "kind": "port",
            "sample": "%d of the same minibatches (same seeds and draws) through the C oracle, "
                      "OpenMP over rows; unique is single-threaded" % done,
            "ms_per_step": cpu_s / done * 1e3,
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
