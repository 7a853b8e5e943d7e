#!/usr/bin/env python3
"""Headline benchmark: forward + backward CSR-by-destination sum SpMM on the
synthetic 2,449,029-node / 61,859,140-edge power-law graph, F=128 fp32, on one
MI355X, through the C ABI of libcxgnn_hip.so.

One step = one forward pass (out = A x over ptr/idx) plus one backward pass
(grad_x = A^T g over the cached transposed CSR).  Graph generation, the
transposition and all allocations of inputs happen before the timed region;
inputs are resident in HBM when timing starts.

Prints ONE JSON line.

``value`` is the metric's *effective* bandwidth: algorithmic bytes of the gather
model (every edge fetches its 4F-byte source row and its 8-byte index; every
output row is written once; ptr is read once) divided by time.  The gather model
charges bytes that the caches serve on a power-law graph, so ``value`` may exceed
the 8 TB/s HBM peak; it is a throughput figure, not a roofline fraction.

``roofline`` is physical: ``achieved`` = bytes that cross the L2 <-> memory-fabric
boundary per launch (``traffic``: rocprofv3 FETCH_SIZE / WRITE_SIZE of the same
launch, calibrated with a plain copy; valid only for the kernel sources whose hash
is recorded next to it) divided by the launch time measured in this run;
``frac`` = achieved / 8 TB/s.  Beside it: the effective (gather-model) rate, the
compulsory-bytes rate, and a *no-reuse control* -- the same kernel on a graph of
the same size with uniform endpoints, where the gather model is (almost) what
the memory really moves -- measured live in this run.

After the timed region the outputs are checked in-process: the adjoint identity
<A x, g> = <x, A^T g> on the timed tensors, and all-ones features -> degrees
(exact) through both passes.
"""
import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "cxgnn-compute_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# Kernel sources the traffic figures below were measured for.
TRAFFIC_SOURCES = ("cxgnn-compute_amd/csrc/spmm.hip", "cxgnn-compute_amd/csrc/cxg_common.hpp")

# Bytes per launch of the aggregation kernel that cross the L2 <-> fabric boundary, from
# rocprofv3 --pmc runs of this file (FETCH_SIZE, WRITE_SIZE scaled by a plain copy of known
# size); the summary named in `profile` holds the counters.  `sources` is sha256[:16] over
# TRAFFIC_SOURCES at the time of the measurement: a figure is only reported for that code.
MEASURED_TRAFFIC = {
    "c3_powerlaw_2.45M_nodes_61.9M_edges_F128": {
        "bytes": 25931085378,
        "sources": "f2a736f9618bebf9",
        "profile": "profiles/spmm_group_kernel_c3_F128_fabric_traffic.md",
    },
}

WORKLOADS = {
    # name: (nodes, undirected pairs, feature width)
    "c3_powerlaw_2.45M_nodes_61.9M_edges_F128": (2449029, 30929570, 128),
    "c2_powerlaw_169k_nodes_2.33M_edges_F128": (169343, 1166243, 128),
}


def sources_hash():
    h = hashlib.sha256()
    for rel in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def spmm_bytes(n_rows, n_edges, feat, index_bytes=8):
    """Gather model: every edge fetches its source row and its index."""
    return n_edges * (4 * feat + index_bytes) + 4 * n_rows * feat + index_bytes * (n_rows + 1)


def spmm_compulsory_bytes(n_rows, n_src_touched, n_edges, feat, index_bytes=8):
    """Perfect reuse: every touched source row and every output row moves once."""
    return 4 * feat * (n_src_touched + n_rows) + index_bytes * (n_edges + n_rows + 1)


def pct(sorted_vals, q):
    if not sorted_vals:
        return None
    k = min(len(sorted_vals) - 1, max(0, int(round(q * (len(sorted_vals) - 1)))))
    return sorted_vals[k]


def summary(vals):
    s = sorted(vals)
    return {"median": round(pct(s, 0.5), 4), "p20": round(pct(s, 0.2), 4), "p80": round(pct(s, 0.8), 4),
            "mean": round(sum(s) / len(s), 4), "n": len(s)}


def cpu_baseline(ptr, idx, ptr_t, idx_t, n_nodes, feat, budget_s=12.0):
    """The reference's own PyTorch SpMM (torch.sparse.mm on a CSR tensor,
    cxgnncomp/codegen/torch_spmm.py:4-9, restated in oracle/pyref.py) on the
    host cores, forward on (ptr, idx) and backward on the transposed CSR, over
    a row prefix of the same graph sized to fit the time budget."""
    import torch
    from oracle import pyref
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(n_nodes, feat, generator=g)
    ptr_c, idx_c = ptr.cpu(), idx.cpu()
    ptrt_c, idxt_c = ptr_t.cpu(), idx_t.cpu()

    def one(rows):
        t0 = time.perf_counter()
        pyref.spmm_torch(x, ptr_c, idx_c, rows)
        pyref.spmm_torch(x, ptrt_c, idxt_c, rows)
        return time.perf_counter() - t0

    rows = max(1, n_nodes // 64)
    t = one(rows)                      # also warms the thread pool
    t = one(rows)
    edges = int(ptr_c[rows]) + int(ptrt_c[rows])
    per_edge = t / max(1, edges)
    total_edges = int(ptr_c[n_nodes]) + int(ptrt_c[n_nodes])
    frac = min(1.0, budget_s / 3.0 / max(per_edge * total_edges, 1e-9))
    rows = max(1, int(n_nodes * frac))
    times = [one(rows) for _ in range(3)]
    t = sorted(times)[1]
    nbytes = (spmm_bytes(rows, int(ptr_c[rows]), feat) + spmm_bytes(rows, int(ptrt_c[rows]), feat))
    return {
        "value": round(nbytes / t / 1e9, 2),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": "torch.sparse.mm(CSR) fwd+bwd on the first %d of %d rows (%d edges) of the same graph, "
                  "median of 3 runs, %.2f s each" % (rows, n_nodes, int(ptr_c[rows]) + int(ptrt_c[rows]), t),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3_powerlaw_2.45M_nodes_61.9M_edges_F128",
                    choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-control", action="store_true",
                    help="skip the no-reuse control (same sizes, uniform endpoints) and the cold-cache passes")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three plain device copies of x (known size) before the timed "
                         "region, to normalise rocprofv3 FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _ops
    from cxgnncomp import synthetic

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n_nodes, n_pairs, feat = WORKLOADS[args.workload]
    ptr, idx = synthetic.powerlaw_symmetric_graph(n_nodes, n_pairs, seed=args.seed, device=dev)
    n_edges = idx.shape[0]
    torch.manual_seed(args.seed)
    x = torch.randn(n_nodes, feat, device=dev)
    grad_out = torch.randn(n_nodes, feat, device=dev)
    graph_t = _ops.transposed(ptr, idx, n_nodes, n_nodes)   # one-time preparation, not timed
    torch.cuda.synchronize()

    if args.copy_probe:
        probe = torch.empty_like(x)
        for _ in range(3):
            probe.copy_(x)
        torch.cuda.synchronize()
        del probe

    zeros9 = (0,) * 9

    def step(events=None):
        if events is not None:
            e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            e0.record()
        out = B.run_spmm_configurable(ptr, idx, x, n_nodes, *zeros9)
        if events is not None:
            e1.record()
        gx = B.run_spmm_configurable_bwd(ptr, idx, x, grad_out, n_nodes, *zeros9)
        if events is not None:
            e2.record()
            events.append((e0, e1, e2))
        return out, gx

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, gx = step(events)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    ms_per_step = elapsed * 1e3 / args.steps
    bytes_pass = spmm_bytes(n_nodes, n_edges, feat)
    bytes_step = 2 * bytes_pass
    flops_step = 2 * n_edges * feat
    value = bytes_step / (ms_per_step * 1e-3) / 1e9

    # Per-launch device time of the aggregation (main kernel + its fix-up) from HIP events
    # recorded on the stream the kernels run on (torch's current stream).
    durs, step_ms = [], []
    for e0, e1, e2 in events:
        durs.append(e0.elapsed_time(e1))
        durs.append(e1.elapsed_time(e2))
        step_ms.append(e0.elapsed_time(e2))
    launch = summary(durs)
    launch_ms = launch["mean"]

    # ---- checks on the timed tensors and on a closed form ----
    # adjoint identity on the outputs of the last timed step: <A x, g> == <x, A^T g>
    lhs = float((out.double() * grad_out.double()).sum())
    rhs = float((x.double() * gx.double()).sum())
    scale = float(out.double().abs().mul(grad_out.double().abs()).sum())
    adj_err = abs(lhs - rhs) / max(scale, 1e-30)
    deg = (ptr[1:] - ptr[:-1]).to(torch.float32)
    deg_t = (graph_t.ptr_t[1:] - graph_t.ptr_t[:-1]).to(torch.float32)
    ones = torch.ones(n_nodes, feat, device=dev)
    out1 = B.run_spmm_configurable(ptr, idx, ones, n_nodes, *zeros9)
    gx1 = B.run_spmm_configurable_bwd(ptr, idx, ones, ones, n_nodes, *zeros9)
    torch.cuda.synchronize()
    ones_ok = bool(torch.equal(out1, deg[:, None].expand(-1, feat))) and \
        bool(torch.equal(gx1, deg_t[:, None].expand(-1, feat)))
    verified = ones_ok and adj_err < 1e-6
    n_src_touched = int((deg_t > 0).sum())
    del ones, out1, gx1
    if not verified:
        sys.exit("bench.py: result check failed (all-ones -> degrees exact: %s, adjoint identity relative "
                 "error %.3e)" % (ones_ok, adj_err))

    # ---- cold-cache passes and the no-reuse control ----
    cold = None
    control = None
    if not args.no_control:
        flush = torch.empty(1 << 28, dtype=torch.float32, device=dev)    # 1 GiB > L2 + last-level cache
        cold_ms = []
        for _ in range(10):
            flush.fill_(1.0)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            B.run_spmm_configurable(ptr, idx, x, n_nodes, *zeros9)
            e1.record()
            torch.cuda.synchronize()
            cold_ms.append(e0.elapsed_time(e1))
        del flush
        cold = summary(cold_ms)
        # same node and edge counts, endpoints uniform: (almost) no source row is gathered twice
        # while it is still cached, so the gather model's bytes are what the memory moves
        u_ptr, u_idx = synthetic.uniform_graph(n_nodes, n_edges, seed=args.seed + 1, device=dev)
        for _ in range(3):
            B.run_spmm_configurable(u_ptr, u_idx, x, n_nodes, *zeros9)
        torch.cuda.synchronize()
        c_ms = []
        for _ in range(20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            u_out = B.run_spmm_configurable(u_ptr, u_idx, x, n_nodes, *zeros9)
            e1.record()
            torch.cuda.synchronize()
            c_ms.append(e0.elapsed_time(e1))
        c = summary(c_ms)
        c_rate = bytes_pass / (c["median"] * 1e-3) / 1e9
        # tie the control to a checked result as well: column sums of A x == in-degree-weighted sums
        u_deg_out = torch.bincount(u_idx, minlength=n_nodes).double()
        want = (u_deg_out[:, None] * x.double()).sum(0)
        got = u_out.double().sum(0)
        c_err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
        if c_err > 1e-6:
            sys.exit("bench.py: control result check failed (column checksum error %.3e)" % c_err)
        control = {
            "workload": "uniform endpoints, %d nodes, %d edges, F=%d (no source-row reuse)" % (n_nodes, n_edges, feat),
            "launch_ms": c,
            "achieved": round(c_rate, 1),
            "frac": round(c_rate / HBM_PEAK_GBS, 4),
            "note": "gather-model bytes / median launch time; ~1.25 GB of source rows against 4 MB of L2 per XCD",
        }
        del u_ptr, u_idx, u_out

    eff = bytes_pass / (launch_ms * 1e-3) / 1e9
    compulsory = spmm_compulsory_bytes(n_nodes, n_src_touched, n_edges, feat)
    meas = MEASURED_TRAFFIC.get(args.workload)
    cur_hash = sources_hash()
    traffic = meas["bytes"] if meas and meas["sources"] == cur_hash else None
    if traffic is not None:
        achieved = traffic / (launch_ms * 1e-3) / 1e9
        basis = "measured L2<->fabric bytes per launch (%s) / launch time of this run" % meas["profile"]
    elif control is not None:
        achieved = None
        basis = "no traffic measurement for these kernel sources (hash %s); see control" % cur_hash
    else:
        achieved = None
        basis = "no traffic measurement for these kernel sources (hash %s)" % cur_hash

    result = {
        "metric": "SpMM fwd+bwd GB/s (% of HBM peak) + GFLOP/s at 61.9M edges, F=128, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "nodes": n_nodes, "edges": n_edges, "feat": feat,
                   "index_dtype": "int64", "op": "sum SpMM forward + transposed-graph backward"},
        "value_definition": "effective GB/s: gather-model bytes / wall time; counts bytes the caches serve, "
                            "so it is not bounded by the HBM peak (see roofline for the physical fraction)",
        "effective_pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "gflops": round(flops_step / (ms_per_step * 1e-3) / 1e9, 1),
        "algorithmic_bytes_per_step": bytes_step,
        "step_ms": summary(step_ms),
        "verified": "all-ones -> degrees exact on out and gx; adjoint identity on the timed tensors, "
                    "relative error %.1e" % adj_err,
        "roofline": {
            "bound": "hbm",
            "kernel": "spmm_group_kernel (+ spmm_fixup_kernel), one cxg_spmm_sum_f32 call",
            "achieved": None if achieved is None else round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": None if achieved is None else round(achieved / HBM_PEAK_GBS, 4),
            "frac_basis": basis,
            "traffic": traffic,
            "kernel_sources_sha256_16": cur_hash,
            "launch_ms": launch_ms,
            "launch_ms_percentiles": launch,
            "cold_launch_ms": cold,
            "algorithmic_bytes_per_launch": bytes_pass,
            "effective": round(eff, 1),
            "effective_frac": round(eff / HBM_PEAK_GBS, 4),
            "compulsory_bytes_per_launch": compulsory,
            "compulsory_frac": round(compulsory / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "control": control,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(ptr, idx, graph_t.ptr_t, graph_t.idx_t, n_nodes, feat)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
