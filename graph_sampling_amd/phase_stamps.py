"""Where the microseconds of a minibatch kernel go: per-phase wall-clock tables.

A measuring aid, not part of the sampling path.  The kernels of the GraphSAGE minibatch carry
marks (GS_STAMP in csrc/) that exist only in a build with -DGS_PHASE_STAMPS: thread 0 of a
workgroup waits for its outstanding memory operations, reads the 100 MHz wall clock, and
appends one record per workgroup to a buffer this script registers.  Build that library once
(`python -m graph_sampling_amd.build --stamps`, here or on any machine with hipcc), then on
the GPU:

    python -m graph_sampling_amd.phase_stamps [--api layers|loop] [--workload 2.45M|111M]

`mean dur` is the average over workgroups of the time between two marks, `crit end` the
latest any workgroup reaches the mark, counted from the launch's first workgroup entry: what
the launch as a whole waits for.  Layers are the three layers of a [15,10,5] minibatch of
1024 seeds.  The marks cost a few hundred nanoseconds each, so the totals here run above the
unmarked kernels' durations in a profiler trace.
"""
import argparse
import ctypes
import os
import sys

import numpy as np


KINDS = {
    "loop": {1: "sample_group_kernel", 2: "table_insert_kernel", 3: "compact_kernel",
             4: "finish_linked_kernel"},
    "layers": {1: "sample_group_kernel<linked>", 5: "rank_linked_kernel"},
}
PHASES = {
    1: ["column id + offsets", "scan of the counts, sum published", "Floyd's selection",
        "look-back (wave 0)", "barrier; first gathers back", "stores (+ table inserts when linked)"],
    2: ["key + length", "compare-and-swap (+ minimum)", "slot number stored"],
    3: ["slot numbers + length", "slot words", "scan of the flags, sum published",
        "look-back (+ keys in flight)", "barrier", "stores"],
    4: ["first index of the item", "rank of it, slot, length", "stores"],
    5: ["slot numbers + counts", "slot words", "scan, sum published, distances stored",
        "look-back (wave 0)", "tile closed", "cross-tile reads, frontier and renamed ids stored"],
}
REC = 16


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--api", default="layers", choices=sorted(KINDS))
    ap.add_argument("--workload", default="2.45M", choices=("2.45M", "111M"))
    ap.add_argument("--minibatches", type=int, default=20)
    args = ap.parse_args()
    import torch
    from . import build, capi, rmat
    if not os.path.exists(build.STAMPS_LIB):
        sys.exit("build the measuring library first: python -m graph_sampling_amd.build --stamps")
    capi.LIB_PATH = build.STAMPS_LIB
    L = capi.lib()
    dev = torch.device("cuda:0")
    nodes, edges = ((2_450_000, 124_000_000) if args.workload == "2.45M"
                    else (111_000_000, 1_600_000_000))
    indptr, indices = rmat.rmat_csc(nodes, edges, seed=0, device=dev, index_dtype=torch.int32)
    cap = 400_000
    buf = torch.zeros((cap + 1) * REC, dtype=torch.int64, device=dev)
    buf[1] = cap
    for tu in ("sampling", "unique"):
        assert getattr(L, "gs_debug_set_stamps_" + tu)(ctypes.c_void_p(buf.data_ptr())) == 0
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    fanouts = (15, 10, 5)
    box = capi.Mailbox()

    if args.api == "loop":
        table = capi.RelabelTable(1 << 21, torch.int32, dev)

        def minibatch(seeds):
            for k in fanouts:
                sp, si, _, _, _ = capi.sample_uniform_fused(indptr, indices, seeds, k, False, seed=1,
                                                            mailbox=box)
                fr, _, _, t2 = capi.relabel_sampled(seeds, sp, si, table, mailbox=box)
                seeds = fr[:box.wait(t2, dev)]
    else:
        bound = 1024 * 16 * 11 * 6
        tables = [capi.RelabelTable(bound, torch.int32, dev) for _ in range(2)]

        def minibatch(seeds):
            _, ticket = capi.sample_layers(indptr, indices, seeds, fanouts, False, seed=1,
                                           mailbox=box, tables=tables)
            box.wait(ticket, dev)

    sets = [torch.randperm(nodes, generator=gen, device=dev)[:1024].to(torch.int32)
            for _ in range(5 + args.minibatches)]
    for s in sets[:5]:
        minibatch(s)
    torch.cuda.synchronize()
    buf[0] = 0
    torch.cuda.synchronize()
    for s in sets[5:]:
        minibatch(s)
    torch.cuda.synchronize()
    n = min(int(buf[0].item()), cap)
    rec = buf[REC:REC * (n + 1)].cpu().numpy().reshape(n, REC).astype(np.int64)
    names = KINDS[args.api]
    print("per-phase wall clock, api=%s, R-MAT %s, [15,10,5] x 1024 seeds, %d minibatches, %d records"
          % (args.api, args.workload, args.minibatches, n))
    # launches: records of one kind, ordered by entry time; a launch ends where the next record
    # enters after every earlier one has left (launches of one kind never overlap on a stream)
    for kind, name in names.items():
        r = rec[rec[:, 0] == kind]
        r = r[np.argsort(r[:, 4], kind="stable")]
        launches, cur, cur_end = [], [], -1
        for row in r:
            nph = int(row[3])
            if cur and row[4] > cur_end:
                launches.append(np.array(cur))
                cur = []
            cur.append(row)
            cur_end = max(cur_end, int(row[4 + nph - 1]))
        if cur:
            launches.append(np.array(cur))
        print("%s: %d launches" % (name, len(launches)))
        for layer in range(3):
            sel = launches[layer::3]
            if not sel:
                continue
            nph = int(sel[0][0, 3])
            crit, mean, dur, recs = np.zeros(nph), np.zeros(nph), 0.0, 0
            for l in sel:
                st = l[:, 4:4 + nph].astype(np.float64)
                t0 = st[:, 0].min()
                crit += (st.max(axis=0) - t0) / 100.0
                mean[1:] += np.diff(st, axis=1).mean(axis=0) / 100.0
                dur += (st[:, nph - 1].max() - t0) / 100.0
                recs += len(l)
            m = len(sel)
            print("  layer %d: %d workgroups reporting, first entry -> last exit %.2f us"
                  % (layer + 1, recs // m, dur / m))
            print("    %-52s %12s %12s" % ("phase", "mean dur us", "crit end us"))
            for p in range(1, nph):
                print("    %-52s %12.2f %12.2f" % (PHASES[kind][p - 1], mean[p] / m, crit[p] / m))


if __name__ == "__main__":
    main()
