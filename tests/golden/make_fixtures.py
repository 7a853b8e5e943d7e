"""Writes tests/golden/fixtures.json: small input/expected-output vectors for the
graph-kernel path.

The reference ships no golden files for this path (its test scripts load external
datasets), so every vector here is either
  * a known-answer case held in the reference's own files -- the all-ones RGCN toy
    of example/prof_rgcn.py:22-51 (31 neighbours x 128 ones x W = ones -> 3968) and
    the reorder_by docstring of cxgnncomp/schedule.py:72-80 -- or
  * a case small enough to be evaluated by hand from the kernels' definitions
    (src/cpp/src/aggr_kernel.cu:3-53, edge_softmax.cu:3-42, stitch_kernel.cu:23-38,
    schedule.py:20-35, schedule.cu:5-63); the expected values below are written out
    as literals or as closed-form expressions of the inputs, not produced by running
    any implementation under test.
Run:  python tests/golden/make_fixtures.py
"""
import json
import math
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def softmax(v):
    m = max(v)
    e = [math.exp(t - m) for t in v]
    s = sum(e)
    return [t / s for t in e]


def leaky(t, slope):
    return max(t, t * slope)


def main():
    fx = {}

    # --- SpMM sum / mean / weighted on a 4-row graph with an empty row -------------
    ptr = [0, 2, 2, 5, 6]
    idx = [1, 3, 0, 0, 2, 3]
    x = [[1.0, 2.0], [10.0, 20.0], [100.0, 200.0], [1000.0, 2000.0]]
    val = [0.5, 2.0, 1.0, -1.0, 3.0, 0.25]
    fx["spmm_small"] = {
        "ptr": ptr, "idx": idx, "x": x, "val": val,
        "sum": [[1010.0, 2020.0], [0.0, 0.0], [102.0, 204.0], [1000.0, 2000.0]],
        "mean": [[505.0, 1010.0], [0.0, 0.0], [34.0, 68.0], [1000.0, 2000.0]],
        "weighted": [[0.5 * 10 + 2 * 1000, 0.5 * 20 + 2 * 2000], [0.0, 0.0],
                     [1 - 1 + 300, 2 - 2 + 600], [250.0, 500.0]],
        # gradient of sum(out * g) w.r.t. x for g = rows of ones: column sums of A
        "bwd_ones": [[2.0, 2.0], [1.0, 1.0], [1.0, 1.0], [2.0, 2.0]],
        "edge_value_degree": [0.5, 0.5, 1.0 / 3, 1.0 / 3, 1.0 / 3, 1.0],
        "spmv_x0": [1010.0, 0.0, 102.0, 1000.0],
    }

    # --- edge softmax, one head, slope 0.2 ----------------------------------------
    att_dst = [[0.5], [0.0], [-1.0], [2.0]]
    att_src = [[1.0], [-2.0], [0.25], [-0.5]]
    slope = 0.2
    out, mask = [], []
    for r in range(4):
        t = [leaky(att_dst[r][0] + att_src[idx[e]][0], slope) for e in range(ptr[r], ptr[r + 1])]
        out += softmax(t) if t else []
        mask += [v > 0 for v in t]
    fx["edge_softmax_small"] = {"ptr": ptr, "idx": idx, "att_dst": att_dst, "att_src": att_src,
                                "slope": slope, "out": [[v] for v in out], "mask": [[m] for m in mask]}

    # --- SDDMM: 3 edges, 2 heads, 2 channels, dst operand shared by the heads -------
    fx["sddmm_small"] = {
        "src": [0, 1, 1], "dst": [1, 0, 1],
        "src_feat": [[[1.0, 2.0], [3.0, 4.0]], [[5.0, 6.0], [7.0, 8.0]]],
        "dst_feat": [[1.0, 10.0], [100.0, 1000.0]],
        "out": [[2100.0, 4300.0], [65.0, 87.0], [6500.0, 8700.0]],
    }

    # --- all-ones RGCN toy (example/prof_rgcn.py:22-51) -----------------------------
    fx["rgcn_all_ones"] = {"num_neighbor": 31, "feat": 128, "num_rel": 1, "expected_value": 31 * 128}

    # --- reorder_by docstring (cxgnncomp/schedule.py:72-80) -------------------------
    fx["reorder_by_doc"] = {
        "ptr": [0, 3, 5, 9], "idx": [0, 1, 2, 3, 4, 5, 6, 7, 8],      # a..i -> 0..8
        "metric": [2, 0, 1],
        "new_ptr": [0, 4, 7, 9], "new_idx": [5, 6, 7, 8, 0, 1, 2, 3, 4],
    }

    # --- neighbor_grouping, thres 4 (schedule.py:20-35) -----------------------------
    fx["neighbor_grouping_small"] = {
        "ptr": [0, 0, 3, 11, 15, 24], "thres": 4,
        "new_ptr": [0, 0, 3, 7, 11, 15, 19, 23, 24],
        "new_target": [0, 1, 2, 2, 3, 4, 4, 4],
    }

    # --- pad_rel, thres 4, 3 relations with counts 5, 4, 0 (stitch_kernel.cu:23-38) --
    # relation 0: 5 % 4 = 1 -> 3 fill slots; relation 1: 4 % 4 = 0 -> none; relation 2: none
    fx["pad_rel_small"] = {
        "count": [5, 4, 0], "thres": 4, "num_rel": 3, "base": 9,
        "rel_in": [0, 1, 0, 1, 0, 1, 0, 1, 0] + [-1] * 9,
        "rel_out": [0, 1, 0, 1, 0, 1, 0, 1, 0] + [0, 0, 0, 3, 3, 3, 3, 3, 3],
        "idx_pad": [-1] * 9,
    }

    # --- rel_schedule, 2 relations, 2 layers (schedule.cu:5-63) ----------------------
    fx["rel_schedule_small"] = {
        "ptr": [0, 2, 3, 3, 6], "idx": [4, 5, 6, 7, 8, 9], "rel": [0, 1, 1, 0, 0, 1],
        "num_node_in_layer": [2, 4, 4], "num_rel": 2,
        "rel0": {"ptr": [0, 1, 3], "idx": [4, 7, 8], "target": [0, 3]},
        "rel1": {"ptr": [0, 1, 2, 3], "idx": [5, 6, 9], "target": [0, 1, 3]},
        "table": [[1, 2], [2, 3]],
    }

    # --- typed linear: 3 rows, 2 relations, K = N = 2 --------------------------------
    fx["typed_linear_small"] = {
        "x": [[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], "types": [1, 0, 1],
        "w": [[[1.0, 0.0], [0.0, 1.0]], [[0.0, 2.0], [3.0, 0.0]]],
        "out": [[6.0, 2.0], [3.0, 4.0], [18.0, 10.0]],
    }

    # --- byte/flop arithmetic held in the reference's notebooks ----------------------
    fx["arithmetic"] = {"mm_flops_test_dup": [128, 256, 2332486, 128 * 256 * 2332486],
                        "expected_mm_flops": 76430901248}

    with open(os.path.join(HERE, "fixtures.json"), "w") as f:
        json.dump(fx, f, indent=1)
    print("wrote", os.path.join(HERE, "fixtures.json"))


if __name__ == "__main__":
    main()
