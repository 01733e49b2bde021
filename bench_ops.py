#!/usr/bin/env python3
"""Timings of the operators around the headline path (one MI355X), one JSON line each.

bench.py measures the GraphSAGE minibatch; this script times the other rows of the scope
table at the sizes of their configurations -- induced-subgraph slicing, format conversions,
weighted sampling with and without replacement, list sampling, the super-batch helpers,
walks, SDDMM, segment and COO sums, row slicing -- through the same C ABI
(graph_sampling_amd/capi.py), with `algorithmic` = the bytes the operator must move at the
least (stated per line) over the median of the timed calls, and four whole samplers (LADIES
and GraphSAGE written against Matrix, as written and through jit.compile) by wall clock.
Timing of the operators: torch.cuda.Event pairs on the current stream, which is the stream the
C ABI is given; a call is all the launches of the operator, host reads included where the
operator has one.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
HBM_PEAK_GBS = 8000.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--nodes", type=int, default=2_450_000)
    ap.add_argument("--edges", type=int, default=124_000_000)
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--only", default="", help="comma-separated operator names")
    args = ap.parse_args()
    import torch
    from graph_sampling_amd import capi, rmat

    if not torch.cuda.is_available():
        print("bench_ops.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    capi.lib()
    dev = torch.device("cuda:0")
    N, E = args.nodes, args.edges
    idt = torch.int32
    b = 4
    indptr, indices = rmat.rmat_csc(N, E, seed=0, device=dev, index_dtype=idt)
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    weights = 1.0 - torch.rand(E, generator=gen, device=dev)
    only = set(x for x in args.only.split(",") if x)

    def rand_ids(n, hi=N):
        return torch.randint(0, hi, (n,), generator=gen, device=dev).to(idt)

    def perm_ids(n):
        return torch.randperm(N, generator=gen, device=dev)[:n].to(idt)

    def run(name, what, fn, bytes_of):
        if only and name not in only:
            return
        for _ in range(2):
            out = fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(args.reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = fn()
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3)
        times.sort()
        t = times[len(times) // 2]
        nbytes, units, unit_name = bytes_of(out)
        print(json.dumps({"op": name, "what": what, "ms": t * 1e3, unit_name: units,
                          "per_s": units / t, "algorithmic_bytes": nbytes,
                          "achieved_GBs": nbytes / t / 1e9,
                          "frac_of_hbm_peak": nbytes / t / 1e9 / HBM_PEAK_GBS}), flush=True)

    # ---- column slice of a third-layer frontier (45k columns) ---------------------------------
    cols45k = perm_ids(45_000)

    def slice45k():
        offsets = capi.slice_count(indptr, cols45k)
        return capi.slice_fill(indptr, indices, cols45k, offsets, int(offsets[-1].item()), False)

    run("slice", "gs_slice_count + gs_slice_fill, 45k columns, with select_index; 16 B per edge",
        slice45k, lambda o: (o[0].numel() * (2 * b + 8) + 45_000 * 32, o[0].numel(), "edges"))

    # ---- induced subgraph: 100k columns, 200k admissible rows ---------------------------------
    c100k, r200k = perm_ids(100_000), perm_ids(200_000)
    D = int(capi.slice_count(indptr, c100k)[-1].item())
    run("col_row_slice", "gs_col_row_slice_*: 100k columns x 200k rows, D = %d edges looked at; "
        "b B per edge looked at (id read; one mark bit), 2b + 16 per edge kept twice (packed, "
        "then placed)" % D,
        lambda: capi.col_row_slice(indptr, indices, c100k, r200k),
        lambda o: (D * b + o[1].numel() * 2 * (2 * b + 16), D, "edges"))

    # ---- row slicing of a column slice (FastGCN layer: keep 512 sampled rows) -----------------
    sp = capi.slice_count(indptr, cols45k)
    nnz = int(sp[-1].item())
    s_idx, s_sel, s_col = capi.slice_fill(indptr, indices, cols45k, sp, nnz, True)
    rows512 = perm_ids(512)
    run("row_slice_coo", "gs_row_slice_coo_*: %d edges, 512 row ids; b B per edge looked at, "
        "3b + 8 per edge kept" % nnz,
        lambda: capi.row_slice_coo(s_idx, s_col, rows512),
        lambda o: (nnz * b + o[0].numel() * (3 * b + 8), nnz, "edges"))

    # ---- weighted sampling of the same slice ---------------------------------------------------
    w_slice = weights[:nnz].contiguous()
    run("sample_weighted", "gs_sample_weighted_fill (A-Res, fanout 10) over the 45k-column slice; "
        "b + 4 B per edge read, 2b + 8 per edge kept",
        lambda: capi.sample_weighted(sp, s_idx, w_slice, None, 10),
        lambda o: (nnz * (b + 4) + 450_000 * (2 * b + 8), nnz, "edges"))
    run("sample_weighted_replace", "gs_sample_weighted_replace (inverse CDF, fanout 10) over the "
        "same slice; 4 B read + 4 B prefix write per edge, 2b + 8 per pick",
        lambda: capi.sample_weighted_replace(sp, s_idx, w_slice, None, 10),
        lambda o: (nnz * 8 + 450_000 * (2 * b + 8), nnz, "edges"))

    # ---- doubly-compressed conversions -----------------------------------------------------------
    run("csc2coo", "gs_csc2coo over the whole graph; 8 B offsets per column + b per edge written",
        lambda: capi.csc2coo(indptr, E, idt),
        lambda o: (E * b + N * 8, E, "edges"))

    # CSC -> CSR of a slice: sort 14M (row, column) pairs by row, stable, with the permutation
    s_rows, s_cols = rand_ids(14_000_000), torch.sort(rand_ids(14_000_000, 45_000)).values.to(idt)
    run("coo2csr_sort", "gs_coo2csc on 14M unsorted edges (stable radix sort by row over 2.45M "
        "rows + offsets + permutation), 3 passes for 22-bit keys: a pass's histogram reads the "
        "8-byte word (key, position) of every edge (the first pass the b-byte key), the pass "
        "itself reads word and value and writes them (the last: value, permutation, key), then "
        "the offsets read the sorted keys",
        lambda: capi.coo2csc(s_rows, s_cols, N, False),
        lambda o: (14_000_000 * ((b + 2 * b + 8 + b) + (8 + 2 * (8 + b)) + (8 + 8 + b + 8 + 2 * b)
                                 + b) + N * 8, 14_000_000, "edges"))

    # ---- super-batch helpers on a third-layer super-batch (64 x 45k columns, 14M edges) -------
    B = 64
    M = 14_000_000
    ptr = (torch.arange(B + 1, device=dev, dtype=torch.int64) * (M // B))
    data = rand_ids(M)
    run("batch_encode", "gs_batch_encode, 14M ids in 64 batches; 2b per id",
        lambda: capi.batch_encode(data, ptr, N),
        lambda o: (M * 2 * b, M, "ids"))
    enc = capi.batch_encode(data, ptr, N)  # fits 32 bits: 64 * 2.45M
    run("batch_decode", "gs_batch_decode (ids and batch numbers); 3b per id",
        lambda: capi.batch_decode(enc, N),
        lambda o: (M * 3 * b, M, "ids"))
    ptr2 = (torch.arange(B + 1, device=dev, dtype=torch.int64) * 1024)
    seeds64 = rand_ids(B * 1024)
    run("batch_concat", "gs_batch_concat_*: 64k seeds ++ 14M ids batch by batch; 3b per id (value "
        "in, value and batch number out)",
        lambda: capi.batch_concat([seeds64, data], [ptr2, ptr]),
        lambda o: ((M + B * 1024) * 3 * b, M + B * 1024, "ids"))
    total, key, total_ptr = capi.batch_concat([seeds64, data], [ptr2, ptr])
    run("batch_split", "gs_batch_split, the inverse; 3b per id",
        lambda: capi.batch_split(total, total_ptr, key, [ptr2, ptr]),
        lambda o: ((M + B * 1024) * 3 * b, M + B * 1024, "ids"))
    run("batch_csr_relabel", "gs_batch_csr_relabel: 64 relabels of (1024 seeds, 218k ids) in one "
        "pass; about 70 B per item (insert, compaction, lookup)",
        lambda: capi.batch_csr_relabel(seeds64, ptr2, data, ptr),
        lambda o: ((M + B * 1024) * 70, M + B * 1024, "items"))
    col14 = rand_ids(M)
    run("batch_coo_relabel", "gs_batch_coo_relabel: the same with both ends of 14M edges renamed",
        lambda: capi.batch_coo_relabel(seeds64, ptr2, data, col14, ptr),
        lambda o: ((M + B * 1024) * 70 + M * (2 * b + 8), M + B * 1024, "items"))
    ids_ptr = (torch.arange(B + 1, device=dev, dtype=torch.int64) * 4000)
    chosen = rand_ids(B * 4000)
    run("coo_filter_batched", "gs_coo_filter_*: 14M edges in 64 batches against 4000 chosen ids per "
        "batch; b B per edge looked at (key read; one mark bit), 4b + 8 per edge kept",
        lambda: capi.coo_filter(data, data, col14, chosen, ptr, ids_ptr),
        lambda o: (M * b + o[0].numel() * (4 * b + 8), M, "edges"))
    run("index_search", "gs_index_search: 14M keys against 256k stored ids; 2b per key",
        lambda: capi.index_search(chosen, data),
        lambda o: (M * 2 * b, M, "keys"))

    # ---- unique / relabel of one large frontier --------------------------------------------------
    big = rand_ids(16_000_000)
    run("unique_relabel", "gs_unique_relabel: 16M ids, relabelled in place; about 70 B per item",
        lambda: capi.unique_relabel([big], [big]),
        lambda o: (16_000_000 * 70, 16_000_000, "items"))

    divisor = torch.rand(N, generator=gen, device=dev) + 0.5
    # ---- walks, SDDMM, segment sum at their configuration sizes ---------------------------------
    starts = rand_ids(1_000_000)
    run("random_walk", "gs_random_walk: 1M walkers x 80 steps on this graph; 28 B per live step",
        lambda: capi.random_walk(indptr, indices, starts, 80, seed=3),
        lambda o: (int((o[1_000_000:] >= 0).sum().item()) * 28,
                   int((o[1_000_000:] >= 0).sum().item()), "steps"))
    if not only or "random_walk_4M_200M" in only:
        # the walk configuration's own graph: R-MAT 4 M nodes / 200 M edges
        w_ptr, w_idx = rmat.rmat_csc(4_000_000, 200_000_000, seed=0, device=dev, index_dtype=idt)
        w_starts = rand_ids(1_000_000, 4_000_000)
        run("random_walk_4M_200M", "gs_random_walk: 1M walkers x 80 steps on R-MAT 4M nodes / 200M "
            "edges (the walk configuration's graph); 28 B per live step",
            lambda: capi.random_walk(w_ptr, w_idx, w_starts, 80, seed=3),
            lambda o: (int((o[1_000_000:] >= 0).sum().item()) * 28,
                       int((o[1_000_000:] >= 0).sum().item()), "steps"))
        del w_ptr, w_idx
    if not only or "metapath_walk" in only:
        # three bipartite relations (1M x 2M nodes, 50M edges each), metapath of 4 repeated 4 times
        rels = [rmat.rmat_csc(2_000_000, 50_000_000, seed=30 + r, device=dev, index_dtype=idt,
                              num_src_nodes=2_000_000) for r in range(3)]
        ptr_tab = torch.tensor([r[0].data_ptr() for r in rels], dtype=torch.int64, device=dev)
        idx_tab = torch.tensor([r[1].data_ptr() for r in rels], dtype=torch.int64, device=dev)
        n_tab = torch.tensor([r[0].numel() - 1 for r in rels], dtype=torch.int64, device=dev)
        path = torch.tensor([0, 1, 2, 1] * 4, dtype=torch.int64, device=dev)
        mstarts = rand_ids(1_000_000, 2_000_000)
        run("metapath_walk", "gs_metapath_walk: 1M walkers x 16 steps over three 50M-edge relations; "
            "28 B per live step",
            lambda: capi.metapath_walk(ptr_tab, idx_tab, n_tab, idt, path, mstarts, seed=4),
            lambda o: (int((o[1_000_000:] >= 0).sum().item()) * 28,
                       int((o[1_000_000:] >= 0).sum().item()), "steps"))
        del rels
    feat = torch.rand(N, 64, generator=gen, device=dev)
    er, ec = rand_ids(8_000_000), rand_ids(8_000_000)
    out_e = torch.empty(8_000_000, 1, device=dev)
    run("sddmm_dot", "gs_sddmm_coo u_dot_v, 64-d fp32 features, 8M random edges; 532 B per edge",
        lambda: capi.sddmm_coo("dot", er, ec, None, feat, feat, out_e, 0, 2, 64, 64, 1, 64, None, None),
        lambda o: (8_000_000 * 532, 8_000_000, "edges"))
    # Divide(divisor, axis=0) on the CSC: out[e] = w[e] / divisor[column of e], scalar per edge
    out_w = torch.empty(E, 1, device=dev)
    run("sddmm_div_csc", "gs_sddmm_csc e_div_v over the whole graph (edge weight / per-column scalar): "
        "4 B read + 4 B written per edge, 12 B per column",
        lambda: capi.sddmm_csc("div", indptr, indices, None, None, weights, divisor, out_w, 1, 2,
                               1, 1, 1, 1, None, None),
        lambda o: (E * 8 + N * 12, E, "edges"))
    # Divide(divisor, axis=1) on the COO form: out[e] = w[e] / divisor[row of e], a random read per edge
    coo_col = capi.csc2coo(indptr, E, idt)
    run("sddmm_div_coo_rows", "gs_sddmm_coo e_div_u over the whole graph (edge weight / scalar of the "
        "edge's row): 4 + b read, 4 written and one random 4-byte read per edge",
        lambda: capi.sddmm_coo("div", indices, coo_col, None, weights, divisor, out_w, 1, 0,
                               1, 1, 1, 1, None, None),
        lambda o: (E * (12 + b), E, "edges"))
    # ---- the layer-wise samplers' picks: 512 of 2.45M rows, by weight and uniformly -------------
    row_prob = torch.rand(N, generator=gen, device=dev)
    row_prob[torch.rand(N, generator=gen, device=dev) < 0.7] = 0.0  # most rows unreachable
    all_rows = torch.arange(N, device=dev, dtype=idt)
    run("list_sample_weighted", "gs_list_sample_weighted: 512 of 2.45M rows without replacement "
        "(70% of the weights zero); 4 B per row (the weight, read once) + 16 B per pick",
        lambda: capi.list_sample_weighted(all_rows, row_prob, 512, seed=3),
        lambda o: (N * 4 + 512 * 16, N, "items"))
    run("list_sample_uniform", "gs_list_sample_uniform: 512 of 2.45M rows without replacement",
        lambda: capi.list_sample_uniform(all_rows, 512, False, seed=3),
        lambda o: (512 * (b + 16), 512, "items"))
    # row probabilities straight off a column slice's COO rows (binned by row, added up in LDS)
    out_p = torch.zeros(N, device=dev)
    run("coo_sum", "gs_coo_sum_binned of w^2 over the rows of a 512-column slice's edges into 2.45M sums",
        lambda: capi.coo_sum_binned(indices[:2_000_000], None, weights[:2_000_000], 2, out_p),
        lambda o: (2_000_000 * (b + 4 + 8), 2_000_000, "edges"))
    coo_cols2m = capi.csc2coo(indptr, E, idt)[:2_000_000]
    out_c = torch.zeros(N, device=dev)
    out_d = torch.empty(2_000_000, device=dev)
    run("e_div_u_sum", "gs_e_div_u_sum over the same 2M edges: w / divisor[row], summed per column",
        lambda: capi.e_div_u_sum(indices[:2_000_000], coo_cols2m, weights[:2_000_000], divisor,
                                 out_d, out_c),
        lambda o: (2_000_000 * (2 * b + 4 + 4 + 4 + 8), 2_000_000, "edges"))
    # ---- the tail of a layer-wise sampler on that slice: node set, kept rows, block values --------
    seeds1k, picks512 = perm_ids(1024), perm_ids(512)
    run("sorted_union", "gs_sorted_union: 1024 seeds + 512 picked rows, sorted and distinct (one "
        "workgroup, LDS); 2b per id",
        lambda: capi.sorted_union(seeds1k, picks512),
        lambda o: (1536 * 2 * b, 1536, "ids"))
    hub_rows = torch.sort(torch.unique(indices[:2_000_000])[:1536]).values.contiguous()
    n_nodes = torch.tensor([hub_rows.numel()], dtype=torch.int64, device=dev)
    picked = capi.coo_pick_rows(indices[:2_000_000], coo_cols2m, hub_rows, n_nodes, hub_rows.numel())
    kept = int(picked[2][1])
    run("coo_pick_rows", "gs_coo_pick_rows: the 2M edges of the slice against 1536 rows (binary "
        "search of the set in LDS; count, scan, fill), %d kept; b B per edge looked at + 4 (its "
        "place, written and read), 3b per edge kept" % kept,
        lambda: capi.coo_pick_rows(indices[:2_000_000], coo_cols2m, hub_rows, n_nodes,
                                   hub_rows.numel()),
        lambda o: (2_000_000 * (b + 8) + kept * 3 * b, 2_000_000, "edges"))
    k_key, k_pos = picked[0][:kept].contiguous(), picked[1][:kept].contiguous()
    num_cols2m = int(coo_cols2m.max()) + 1
    run("coo_block_values", "gs_coo_block_values: those kept edges put in block order column by "
        "column (counting sort in LDS) with value = w / divisor[row]; 2b read, b + 4 + 8 "
        "gathered, b + 4 written per kept edge, 8 B per column",
        lambda: capi.coo_block_values(k_key, k_pos, hub_rows.numel(), indices[:2_000_000],
                                      weights[:2_000_000], divisor, num_cols2m),
        lambda o: (kept * (4 * b + 16) + num_cols2m * 8, kept, "edges"))

    out_nrm = torch.empty(E, device=dev)
    run("segment_normalize", "gs_segment_normalize over every column of the graph; 4 B read twice + "
        "4 B written per edge, 16 B per column",
        lambda: capi.segment_normalize(indptr, None, weights, out_nrm),
        lambda o: (E * 12 + N * 16, E, "edges"))
    keep_rows = torch.randperm(N, generator=gen, device=dev)[:200_000].to(idt)
    run("row_slice_csc", "gs_row_slice_csc_*: the whole graph cut down to 200k of its rows (mark, scan "
        "of the tile counts, compact); b B per edge looked at, 4b + 8 per edge kept (new id packed and "
        "placed, column, position)",
        lambda: capi.row_slice_csc(indptr, indices, keep_rows, True),
        lambda o: (E * b + int(o[2].numel()) * (4 * b + 8), E, "edges"))
    out_n = torch.empty(N, device=dev)
    run("segment_sum", "gs_segment_sum of w^2 over every column of the graph; 4 B per edge + 20 B "
        "per column",
        lambda: capi.segment_sum(indptr, None, None, weights, 2, out_n),
        lambda o: (E * 4 + N * 20, E, "edges"))

    # ---- whole samplers through the Matrix layer (wall clock, device drained around each) -------
    import graph_sampling_amd as gs
    from graph_sampling_amd import jit

    def flow(name, what, fn, units_of, unit_name):
        if only and name not in only:
            return
        for _ in range(3):
            out = fn()
        times = []
        for _ in range(max(args.reps, 10)):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = fn()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        times.sort()
        t = times[len(times) // 2]
        units = units_of(out)
        print(json.dumps({"op": name, "what": what, "ms": t * 1e3, unit_name: units,
                          "per_s": units / t}), flush=True)

    A = gs.Matrix().load_csc(indptr, indices, weights)

    def ladies(A, seeds, fanouts):  # the sampler of examples/ladies/ladies_raw.py:8-27
        ret = []
        for fanout in fanouts:
            U = A[:, seeds]
            prob = U.sum(axis=1, powk=2)
            selected, _ = torch.ops.gs_ops.list_sampling_with_probs(U.row_ids(unique=False), prob,
                                                                    fanout, False)
            nodes = torch.cat((seeds, selected)).unique()
            subU = U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0)
            seeds = subU.all_indices()
            ret.insert(0, subU.to_dgl_block())
        return seeds, ret

    def graphsage(A, seeds, fanouts):  # written unfused, as examples/graphsage does before jit
        ret = []
        for k in fanouts:
            sub = A[:, seeds].columnwise_sampling(k, False)
            seeds = sub.all_indices()
            ret.insert(0, sub.to_dgl_block())
        return seeds, ret

    seeds512 = torch.randperm(N, generator=gen, device=dev)[:512].to(idt)
    seeds1024 = torch.randperm(N, generator=gen, device=dev)[:1024].to(idt)
    edges_of = lambda o: sum(blk.num_edges() for blk in o[1])
    flow("flow_ladies", "LADIES, 2 layers of 512 picks from 512 seeds (slice, row sums of w^2 over "
         "2.45M rows, weighted pick, row slice, divide, normalise, relabel)",
         lambda: ladies(A, seeds512, [512, 512]), edges_of, "edges")
    if not only or "config3" in only:
        # the layer-wise sampler's configuration as a line of its own, in the shape of bench.py's:
        # fresh seeds every step, the steps back to back, one synchronisation on either side
        steps, warm = max(args.reps, 10) * 5, 5
        sets = [torch.randperm(N, generator=gen, device=dev)[:512].to(idt)
                for _ in range(warm + steps)]
        for s_ in sets[:warm]:
            ladies(A, s_, [512, 512])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        block_edges = 0
        for s_ in sets[warm:]:
            block_edges += edges_of(ladies(A, s_, [512, 512]))
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        print(json.dumps({
            "metric": "block edges/sec, LADIES 2 layers x 512 weighted picks, batch 512",
            "value": block_edges / dt, "unit": "edges/s", "n_gpus": 1, "steps": steps,
            "warmup": warm, "ms_per_step": dt / steps * 1e3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "int32 ids, fp32 weights",
            "data": "synthetic R-MAT (a=.57,b=.19,c=.19), generated on device, seed 0",
            "config": {"workload": "rmat-%.2fM-%dM ladies" % (N / 1e6, E // 1_000_000),
                       "batch": 512, "picks_per_layer": [512, 512],
                       "api": "gs.Matrix: A[:, seeds], sum(axis=1, powk=2), "
                              "list_sampling_with_probs, U[nodes, :], divide, normalize, "
                              "all_indices, to_dgl_block (examples/ladies/ladies_raw.py:8-27)"}}),
              flush=True)
    ladies_c = jit.compile(ladies, (A, seeds512, [512, 512]))
    flow("flow_ladies_compiled", "the same sampler through jit.compile",
         lambda: ladies_c(A, seeds512, [512, 512]), edges_of, "edges")
    # the GraphSAGE examples load the adjacency alone (examples/graphsage/graphsage_fused.py:23-26):
    # no edge data follows the samples
    P = gs.Matrix().load_csc(indptr, indices)
    flow("flow_graphsage_unfused", "GraphSAGE [15,10,5], 1024 seeds, written as slice -> sample -> "
         "all_indices -> block through the Matrix layer",
         lambda: graphsage(P, seeds1024, [15, 10, 5]), edges_of, "edges")
    sage_c = jit.compile(graphsage, (P, seeds1024, [15, 10, 5]))
    flow("flow_graphsage_compiled", "the same sampler through jit.compile (its three layers as one "
         "chain call)",
         lambda: sage_c(P, seeds1024, [15, 10, 5]), edges_of, "edges")
    flow("flow_graphsage_compiled_weights", "the compiled sampler on the graph with edge weights "
         "(the weights follow the samples: layer by layer)",
         lambda: sage_c(A, seeds1024, [15, 10, 5]), edges_of, "edges")


if __name__ == "__main__":
    main()
