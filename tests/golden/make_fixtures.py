"""Writes the golden fixtures of this directory.

reference_vectors.json   inputs and expected outputs of the reference's own gtest cases
                         (tests/*.cc of czkkkkkk/graph_sampling), transcribed as data.  Every
                         entry names the reference test it comes from.
replay_small.npz         a 512-node R-MAT graph, replay draws and the CPU oracle's outputs for
                         them (sampling with both algorithms, weighted sampling, walks,
                         unique/relabel).  The GPU tests compare against these arrays, so a
                         change of either implementation shows up as a diff of committed data.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)


def reference_vectors():
    a20 = {"indptr": (np.arange(21) * 5).tolist(), "indices": list(range(100))}
    g12 = {"indptr": [0] * 10 + [0, 2, 4], "indices": [1, 3, 1, 3]}
    return {
        "graph_20x5": a20,
        "graph_12col": g12,
        "colwise_slicing_test1": {  # tests/test_colwise_slicing.cc:7-20
            "cols": [0, 1, 2], "indptr": (np.arange(4) * 5).tolist(), "indices": list(range(15))},
        "colwise_sampling_test1": {  # tests/test_colwise_sampling.cc:7-20 (fanout 6 >= degree 5)
            "fanout": 6, "replace": False, "indptr": a20["indptr"], "indices": a20["indices"]},
        "colwise_sampling_test2": {  # :22-37
            "fanout": 6, "replace": True, "indptr": (np.arange(21) * 6).tolist(), "max_unique": 100},
        "colwise_sampling_test3": {  # :39-53
            "fanout": 4, "replace": True, "indptr": (np.arange(21) * 4).tolist(), "max_unique": 100},
        "slicing_relabel_test1": {  # tests/test_relabel.cc:7-26
            "cols": [1, 2, 3], "num_rows": 15, "num_cols": 3,
            "indptr": (np.arange(4) * 5).tolist(), "indices": list(range(15))},
        "rowwise_slicing_test1": {  # tests/test_rowwise_slicing.cc:7-20
            "rows": list(range(0, 100, 5)), "indptr": list(range(21)), "indices": list(range(20))},
        "list_sampling": {  # tests/test_listsampling.cc:7-40
            "n": 1000, "identity_k": 2000, "replace_k": 2000, "distinct_k": 999},
        "graph_sum_test1": {"axis": 0, "powk": 1, "expected": [5.0] * 20},   # test_graph_compute.cc:8-20
        "graph_sum_test2": {"data": list(range(1, 6)) * 20, "powk": 1, "expected": [15.0] * 20},  # :22-37
        "graph_sum_test3": {"powk": 2, "expected": [5.0] * 20},              # :39-51
        "graph_sum_test4": {"data": list(range(1, 6)) * 20, "powk": 2, "expected": [55.0] * 20},  # :53-68
        "graph_sum_test5": {  # :70-91 row sums (CSR) of the 12-column graph, data 3..6
            "data": [3, 4, 5, 6], "expected": [0, 8, 0, 10] + [0] * 8},
        "graph_div_test2": {  # :150-165: ones / divisor[col]
            "divisor": list(range(1, 21))},
        "graph_normalize_test4": {  # :243-263: slice cols 10,11 then row-normalise
            "data": [3, 4, 5, 6], "expected": [3 / 8, 4 / 10, 5 / 8, 6 / 10]},
        "sddmm_add_test1": {"n": 100},  # tests/test_sddmm.cc:7-22: coo row=col=arange, out = 2*arange
        "sddmm_add_test2": {"rhs_n": 20},  # :24-37: lhs[row] + rhs[col]
        "csc2csr_test3": {  # tests/test_format_transform.cc:54-74
            "indptr": [0, 0, 2, 2] + [4] * 9, "indices": [10, 11, 10, 11], "e_ids": [0, 2, 1, 3]},
        "csc2dcsr_test1": {"valid_rows": [1, 3], "indices": [10, 11, 10, 11]},  # :100-116
        "hetero_walk_one_path": {  # tests/test_hetero_random_walk.cc:29-71
            "follow": {"indptr": [0, 0, 1, 2, 3], "indices": [0, 1, 2]},
            "view": {"indptr": [0, 1, 2, 3], "indices": [0, 1, 2]},
            "metapath": ["view", "follow", "follow"], "seeds": [2, 1],
            "trace_step_major": [2, 1, 2, 1, 1, 0, 0, -1]},
        "hetero_walk_multi_path": {  # :74-120
            "follow": {"indptr": [0, 0, 1, 2, 3], "indices": [0, 1, 2]},
            "view": {"indptr": [0, 1, 3, 5], "indices": [0, 0, 1, 2, 3]},
            "metapath": ["view", "follow", "follow"], "seeds": [2, 2, 1, 1, 0]},
        "philox4x32_10_kat": [  # Random123 kat_vectors (philox4x32 10 rounds)
            {"ctr": [0, 0, 0, 0], "key": [0, 0],
             "out": [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]},
            {"ctr": [0xffffffff] * 4, "key": [0xffffffff] * 2,
             "out": [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]},
            {"ctr": [0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], "key": [0xa4093822, 0x299f31d0],
             "out": [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]},
        ],
    }


def replay_small():
    from oracle import oracle as O
    from tests.util import rmat_csc_np, u32_draws
    indptr, indices = rmat_csc_np(512, 4096, seed=42)
    rng = np.random.default_rng(7)
    cols = rng.integers(0, 512, size=256).astype(np.int64)
    cols[:3] = np.argsort(np.diff(indptr))[-3:]
    probs = (1.0 - rng.random(indices.size)).astype(np.float32)
    out = {"indptr": indptr, "indices": indices, "cols": cols, "probs": probs}
    for name, algo in (("floyd", O.ALGO_AUTO), ("reservoir", O.ALGO_RESERVOIR)):
        _, rp = O.sample_count(indptr, cols, 5, False, want_replay_ptr=True, algo=algo)
        draws = u32_draws(int(rp[-1]), 100 + algo)
        r = O.sample_uniform(indptr, indices, cols, 5, False, replay=draws, with_coo=False, algo=algo)
        out["%s_replay_ptr" % name] = rp
        out["%s_draws" % name] = draws
        out["%s_sub_indptr" % name] = r[0]
        out["%s_sub_indices" % name] = r[2]
        out["%s_select_index" % name] = r[3]
    rp = O.weighted_replay_ptr(indptr, cols, 4)
    draws = u32_draws(int(rp[-1]), 200)
    r = O.sample_weighted(indptr, indices, probs, cols, 4, replay=draws, with_coo=False)
    out.update(weighted_replay_ptr=rp, weighted_draws=draws, weighted_sub_indptr=r[0],
               weighted_sub_indices=r[2], weighted_select_index=r[3])
    seeds = rng.integers(0, 512, size=128).astype(np.int64)
    draws = u32_draws(128 * 6, 300)
    out.update(walk_seeds=seeds, walk_draws=draws,
               walk_trace=O.random_walk(indptr, indices, seeds, 6, replay=draws))
    frontier, rel = O.relabel([cols, out["floyd_sub_indices"]], [out["floyd_sub_indices"]])
    out.update(relabel_frontier=frontier, relabel_rows=rel[0])
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "reference_vectors.json"), "w") as f:
        json.dump(reference_vectors(), f, indent=1, sort_keys=True)
    np.savez_compressed(os.path.join(HERE, "replay_small.npz"), **replay_small())
    print("wrote", os.listdir(HERE))
