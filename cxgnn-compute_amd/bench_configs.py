#!/usr/bin/env python3
"""Per-operator throughput on the five benchmark configurations (one JSON line per
measurement).  ``bench.py`` at the repository root reports the headline metric;
this script is the wider table: every op of the graph-kernel path at the shape it
has in each configuration, as milliseconds, effective GB/s (algorithmic bytes of
the gather model / time), GFLOP/s and fraction of the 8 TB/s HBM peak (or of the
matrix-core peak for the typed GEMM).

Timing: HIP events around every call; ``ms`` is the median of the timed calls,
``p20_ms`` / ``p80_ms`` the spread.  ``--cold`` overwrites a 1 GiB buffer before
every timed call so that nothing of the previous call is left in the L2 or the
256 MB last-level cache; the default is warm (back-to-back calls).
``--cpu-baseline`` adds, per configuration, the same ops in plain PyTorch on the
host cores (the restatements of the reference's own PyTorch paths kept with the
CPU oracle), on bounded samples of the same graphs.

Usage: python bench_configs.py [--configs c1,c2,c3,c4,c5] [--iters 10] [--cold] [--cpu-baseline]
       python bench_configs.py --configs c5 --c5-steps 20 [--c5-fresh]    (only the sampled-batch training step)
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

import torch  # noqa: E402

HBM = 8000.0          # GB/s
MFMA_F32 = 157300.0   # GFLOP/s
MFMA_BF16 = 2500000.0


COLD = False
CPU_BASELINE = False
C5_STEPS = 0
C5_FRESH = False
_flush = None
_last_spread = None


def timeit(fn, iters, warm=3):
    """Median milliseconds of ``iters`` calls, each bracketed by its own HIP events."""
    global _flush, _last_spread
    for _ in range(warm):
        fn()
    if COLD and _flush is None:
        _flush = torch.empty(1 << 28, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    evs = []
    for _ in range(iters):
        if COLD:
            _flush.zero_()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        evs.append((s, e))
    torch.cuda.synchronize()
    ts = sorted(s.elapsed_time(e) for s, e in evs)
    _last_spread = (ts[int(0.2 * (len(ts) - 1))], ts[int(round(0.8 * (len(ts) - 1)))])
    return ts[len(ts) // 2]


def report(cfg, op, ms, nbytes=None, flops=None, peak_flops=None, note=""):
    global _last_spread
    rec = {"config": cfg, "op": op, "ms": round(ms, 4)}
    if _last_spread is not None:
        rec["p20_ms"], rec["p80_ms"] = round(_last_spread[0], 4), round(_last_spread[1], 4)
        _last_spread = None
    rec["cache"] = "cold" if COLD else "warm"
    if nbytes:
        gbs = nbytes / ms / 1e6
        rec["eff_GBps"] = round(gbs, 1)
        rec["frac_hbm"] = round(gbs / HBM, 4)
    if flops:
        gf = flops / ms / 1e6
        rec["GFLOPps"] = round(gf, 1)
        if peak_flops:
            rec["frac_mfma"] = round(gf / peak_flops, 4)
    if note:
        rec["note"] = note
    print(json.dumps(rec), flush=True)


def cpu_report(cfg, op, fn, sample, nbytes=None, repeats=3):
    """One warm-up call and ``repeats`` timed calls of a host-side PyTorch restatement."""
    import time
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    fn()
    ts = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        fn()
        ts.append((time.perf_counter() - t0) * 1e3)
    ms = sorted(ts)[len(ts) // 2]
    rec = {"config": cfg, "op": op, "cpu_ms": round(ms, 3), "cores": cores, "sample": sample}
    if nbytes:
        rec["cpu_eff_GBps"] = round(nbytes / ms / 1e6, 2)
    print(json.dumps(rec), flush=True)


def spmm_bytes(rows, edges, row_floats, val_floats=0):
    return edges * (4 * row_floats + 8 + 4 * val_floats) + 4 * rows * row_floats + 8 * (rows + 1)


def bench_aggregation(cfg, ptr, idx, n_dst, n_src, feat, iters, weighted=True):
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _ops
    E = int(ptr[n_dst])
    x = torch.randn(n_src, feat, device="cuda")
    g = torch.randn(n_dst, feat, device="cuda")
    gt = _ops.transposed(ptr, idx, n_dst, n_src)
    z = (0,) * 9
    report(cfg, "spmm_sum_fwd F=%d" % feat, timeit(lambda: B.run_spmm_configurable(ptr, idx, x, n_dst, *z), iters),
           spmm_bytes(n_dst, E, feat), E * feat)
    report(cfg, "spmm_sum_bwd F=%d" % feat,
           timeit(lambda: B.run_spmm_configurable_bwd(ptr, idx, x, g, n_dst, *z), iters),
           spmm_bytes(n_src, E, feat), E * feat)
    report(cfg, "spmm_mean_fwd F=%d" % feat, timeit(lambda: _ops.spmm(ptr, idx, x, n_dst, mean=True), iters),
           spmm_bytes(n_dst, E, feat), E * feat)
    if weighted:
        val = B.edge_value_degree(ptr, n_dst, idx.shape[0])
        report(cfg, "spmm_weighted_fwd(1/deg) F=%d" % feat,
               timeit(lambda: _ops.spmm(ptr, idx, x, n_dst, val=val), iters),
               spmm_bytes(n_dst, E, feat, 1), 2 * E * feat)
        report(cfg, "spmm_weighted_bwd F=%d" % feat,
               timeit(lambda: _ops.spmm(gt.ptr_t, gt.idx_t, g, n_src, val=val, val_perm=gt.perm), iters),
               spmm_bytes(n_src, E, feat, 1) + 8 * E, 2 * E * feat)


def cpu_spmm(cfg, ptr, idx, n_src, feat, rows):
    """torch.sparse.mm on the first ``rows`` rows (cxgnncomp/codegen/torch_spmm.py:4-9)."""
    from oracle import pyref
    p, i = ptr[:rows + 1].cpu(), idx[:int(ptr[rows])].cpu()
    x = torch.randn(n_src, feat)
    e = int(p[-1])
    cpu_report(cfg, "spmm_sum_fwd F=%d torch.sparse.mm" % feat, lambda: pyref.spmm_torch(x, p, i, rows),
               "first %d rows, %d edges" % (rows, e), spmm_bytes(rows, e, feat))


def c1(iters):
    from cxgnncomp import synthetic as S
    ptr, idx = S.uniform_graph(10000, 100000, device="cuda")
    bench_aggregation("c1", ptr, idx, 10000, 10000, 64, iters)
    if CPU_BASELINE:
        cpu_spmm("c1", ptr, idx, 10000, 64, 10000)


def c2(iters):
    from cxgnncomp import synthetic as S
    ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, device="cuda")
    for f in (128, 256):
        bench_aggregation("c2", ptr, idx, 169343, 169343, f, iters)
        if CPU_BASELINE:
            cpu_spmm("c2", ptr, idx, 169343, f, 169343)
    # the configuration's model: 3 GCN layers 128 -> 256 -> 256 -> 40, BatchNorm + ReLU between
    import cxgnncomp
    cxgnncomp.set_timers()                       # MyGCNConv brackets its phases with TimerOP, as upstream
    n = 169343
    x = torch.randn(n, 128, device="cuda")
    for normalize, own_bn in ((False, True), (True, True), (False, False)):
        convs = [cxgnncomp.MyGCNConv(128, 256, normalize).cuda(), cxgnncomp.MyGCNConv(256, 256, normalize).cuda(),
                 cxgnncomp.MyGCNConv(256, 40, normalize).cuda()]
        # between the layers, as GNN._between: the library's BatchNorm1d with the ReLU fused, or torch's own
        bn_cls = cxgnncomp.BatchNorm1d if own_bn else torch.nn.BatchNorm1d
        bns = [bn_cls(256).cuda(), bn_cls(256).cuda()]
        xg = x.clone().requires_grad_(True)
        gout = torch.randn(n, 40, device="cuda") / 16     # the gradient a loss would hand back

        def step():
            xg.grad = None
            h = xg
            for li, conv in enumerate(convs):
                h = conv(h, ptr, idx, n)
                if li < 2:
                    h = bns[li](h, relu=True) if own_bn else torch.relu(bns[li](h))
            h.backward(gout)
        report("c2", "3-layer GCN fwd+bwd, %s aggregation%s" % ("1/deg-weighted" if normalize else "sum",
                                                                "" if own_bn else ", torch.nn.BatchNorm1d + relu"),
               timeit(step, iters))
    bn = cxgnncomp.BatchNorm1d(256).cuda()
    hb = torch.randn(n, 256, device="cuda").requires_grad_(True)
    gb = torch.randn(n, 256, device="cuda")
    report("c2", "BatchNorm1d + ReLU forward, [169343, 256]", timeit(lambda: bn(hb, relu=True), iters), 2 * 3 * n * 256 * 4 // 3)
    yb = bn(hb, relu=True)
    report("c2", "BatchNorm1d + ReLU backward, [169343, 256]",
           timeit(lambda: torch.autograd.grad(yb, hb, gb, retain_graph=True), iters), 5 * n * 256 * 4)
    del bn, hb, gb, yb
    del convs, bns, xg
    # the remaining aggregation entry points of the backend on the same graph, F = 128
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _ops
    E, F = idx.shape[0], 128
    xe = torch.randn(E, F, device="cuda")
    dest = _ops.csr_row_ids(ptr, n, E)
    report("c2", "gather (edge -> node sum, rows grouped by destination once) F=128", timeit(lambda: B.gather(xe, dest, n), iters),
           E * (4 * F + 8) + 8 * n * F, E * F)
    del xe
    mask = (torch.rand(E, device="cuda") < 0.5)
    out = torch.zeros(n, F, device="cuda")
    report("c2", "selective_aggr (half of the edges masked) F=128",
           timeit(lambda: B.selective_aggr(x, ptr, idx, mask, out, n), iters),
           spmm_bytes(n, E, F) // 2 + E + 4 * n * F, E * F)
    gsel = torch.zeros(n, F, device="cuda")
    report("c2", "selective_aggr_bwd F=128", timeit(lambda: B.selective_aggr_bwd(out, ptr, idx, mask, gsel, n), iters),
           spmm_bytes(n, E, F) // 2 + 9 * E + 4 * n * F, E * F)
    import cxgnncomp
    gp, gtar = cxgnncomp.neighbor_grouping(ptr, 32)
    out.zero_()
    report("c2", "target_aggr over neighbor groups of 32 (%d groups) F=128" % gtar.shape[0],
           timeit(lambda: B.target_aggr(x, gp, idx, gtar, out, gtar.shape[0]), iters),
           spmm_bytes(gtar.shape[0], E, F) + 8 * gtar.shape[0], 2 * E * F)
    xs = torch.randn(n, device="cuda")
    report("c2", "spmv (unit values)", timeit(lambda: B.spmv(ptr, idx, xs, n), iters), E * 12 + 12 * n, E)
    report("c2", "edge_value_degree", timeit(lambda: B.edge_value_degree(ptr, n, E), iters), 8 * n + 4 * E)
    p32, i32 = ptr.int(), idx.int()
    report("c2", "GSpMM_u MAX (int32 CSR) F=128", timeit(lambda: B.GSpMM_u(p32, i32, x, B.REDUCEOP.MAX), iters),
           E * (4 * F + 4) + 4 * n * F, E * F)
    ev = torch.rand(E, device="cuda")
    report("c2", "GSpMM_u_e SUM x MUL (int32 CSR) F=128",
           timeit(lambda: B.GSpMM_u_e(p32, i32, ev, x, B.REDUCEOP.SUM, B.COMPUTEOP.MUL), iters),
           E * (4 * F + 8) + 4 * n * F, 2 * E * F)


def c3(iters):
    import cxgnncomp_backend as B
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    N = 2449029
    ptr, idx = S.powerlaw_symmetric_graph(N, 30929570, device="cuda")
    E = idx.shape[0]
    bench_aggregation("c3", ptr, idx, N, N, 128, iters, weighted=False)
    H, C = 4, 64
    att_s = torch.randn(N, H, device="cuda")
    att_d = torch.randn(N, H, device="cuda")
    ev, mask = _ops.edge_softmax_fwd(ptr, idx, att_d, att_s, E, 0.2)
    sm_bytes = E * (8 + 4 * H) + 4 * E * H + E * H + 4 * N * H + 8 * (N + 1)
    report("c3", "edge_softmax_fwd H=4", timeit(lambda: _ops.edge_softmax_fwd(ptr, idx, att_d, att_s, E, 0.2), iters),
           sm_bytes, 6 * E * H)
    gev = torch.randn(E, H, device="cuda")
    gt = _ops.transposed(ptr, idx, N, N)

    rows_t = _ops.rows32_transposed(gt)

    def sm_bwd():
        g_dst, t_edge = _ops.edge_softmax_bwd(ptr, ev, mask, gev, N, 0.2)
        return _ops.narrow_gather_sum(gt.ptr_t, gt.perm, t_edge, N, rows32=rows_t)
    report("c3", "edge_softmax_bwd H=4 (row pass + transposed gather)", timeit(sm_bwd, iters),
           E * H * (4 + 4 + 1 + 4) + E * (8 + 4 * H) + 8 * N * H, 6 * E * H)
    x = torch.randn(N, H, C, device="cuda") / 8
    g = torch.randn(N, H, C, device="cuda") / 8
    report("c3", "spmm_multihead_fwd H=4 C=64", timeit(lambda: _ops.spmm(ptr, idx, x, N, val=ev), iters),
           spmm_bytes(N, E, H * C, H), 2 * E * H * C)
    # the GAT layer's forward aggregation when its input has 128 columns: the input rows gathered once
    # under the four edge weights (out [N, 4, 128]), then one 128 -> 64 product per head
    x_in = x.view(N, H * C)[:, :128].contiguous()
    report("c3", "spmm, one gathered 128-float row under H=4 weights (out [N, 4, 128])",
           timeit(lambda: _ops.spmm_weighted_heads(ptr, idx, ev, x_in, N), iters),
           E * (4 * 128 + 8 + 4 * H) + 4 * N * H * 128 + 8 * (N + 1), 2 * E * H * 128)
    from cxgnncomp_backend import _typed
    aggr, w_heads = torch.randn(N, H, 128, device="cuda") / 8, torch.randn(H * C, 128, device="cuda") / 8
    b_heads = torch.randn(H * C, device="cuda")
    report("c3", "per-head products [N, 4, 128] x 4 [128, 64] + bias after that aggregation",
           timeit(lambda: _typed.dense_linear_heads(aggr, w_heads, b_heads), iters), 4 * N * H * (128 + C), 2 * N * H * 128 * C)
    del x_in, aggr, w_heads, b_heads
    import cxgnncomp_backend as B
    report("c3", "spmm_multihead PreReduce H=4 C=64 (heads summed inside the kernel, out [N, 64])",
           timeit(lambda: B.spmm_multihead(ptr, idx, ev, x, N, B.SPMM_MULTIHEAD_SCHEDULE.PreReduce), iters),
           E * (4 * H * C + 8 + 4 * H) + 4 * N * C + 8 * (N + 1), 2 * E * H * C)
    report("c3", "the same as two passes (Naive, then a sum over the heads)",
           timeit(lambda: _ops._C.head_sum(B.spmm_multihead(ptr, idx, ev, x, N, B.SPMM_MULTIHEAD_SCHEDULE.Naive)), iters),
           E * (4 * H * C + 8 + 4 * H) + 4 * N * C + 8 * (N + 1), 2 * E * H * C)
    from cxgnncomp.graph_kernel import SpMMValOP
    xv, evv = x.clone().requires_grad_(True), ev.clone().requires_grad_(True)

    def valop_step():
        xv.grad = None
        evv.grad = None
        SpMMValOP.apply(xv, ptr, idx, evv, N).backward(g)
    report("c3", "SpMMValOP H=4 C=64 forward + backward (input and edge-value gradients)", timeit(valop_step, max(2, iters // 3)))
    del xv, evv
    report("c3", "spmm_multihead_bwd H=4 C=64",
           timeit(lambda: _ops.spmm(gt.ptr_t, gt.idx_t, g, N, val=ev, val_perm=gt.perm), iters),
           spmm_bytes(N, E, H * C, H) + 8 * E, 2 * E * H * C)
    report("c3", "sddmm_csr (edge-value grad) H=4 C=64", timeit(lambda: _ops.sddmm_csr(ptr, idx, x, g, N), iters),
           E * (4 * H * C + 8) + 4 * N * H * C + 4 * E * H, 2 * E * H * C)
    gev = torch.empty(E, H, device="cuda")
    report("c3", "spmm_multihead_bwd + edge-value grad in one pass (spmm_dot) H=4 C=64",
           timeit(lambda: _ops.spmm_dot(gt.ptr_t, gt.idx_t, g, N, ev, gt.perm, x, gev), iters),
           spmm_bytes(N, E, H * C, H) + 8 * E + 4 * N * H * C + 4 * E * H, 4 * E * H * C)
    report("c3", "the same with the edge-value grad left in the reversed graph's edge order (contiguous stores; the GAT layer's path)",
           timeit(lambda: _ops.spmm_dot(gt.ptr_t, gt.idx_t, g, N, ev, gt.perm, x, gev, dot_at_edge=True), iters),
           spmm_bytes(N, E, H * C, H) + 8 * E + 4 * N * H * C + 4 * E * H, 4 * E * H * C)
    inv = _ops.inverse_perm_transposed(gt)
    report("c3", "edge_softmax_bwd row pass H=4, gradient in edge order",
           timeit(lambda: _ops.edge_softmax_bwd(ptr, ev, mask, gev, N, 0.2), iters),
           E * (4 * H * 3 + H) + 8 * N + 4 * N * H, 6 * E * H)
    report("c3", "edge_softmax_bwd row pass H=4, gradient read through the inverse permutation (the GAT layer's path)",
           timeit(lambda: _ops.edge_softmax_bwd(ptr, ev, mask, gev, N, 0.2, grad_pos=inv), iters),
           E * (4 * H * 3 + H + 8) + 8 * N + 4 * N * H, 6 * E * H)
    del gev, inv
    dst = _ops.csr_row_ids(ptr, N, E)
    out = torch.empty(E, H, device="cuda")
    report("c3", "sddmm_coo H=4 C=64", timeit(lambda: _ops.sddmm_coo(idx, dst, x, g, out, E), iters),
           E * (8 * H * C + 16) + 4 * E * H, 2 * E * H * C)
    # single-head F=128 (several edges per gather step), same graph
    x1, g1 = x.view(N, H * C)[:, :128].contiguous(), g.view(N, H * C)[:, :128].contiguous()
    report("c3", "sddmm_csr H=1 C=128", timeit(lambda: _ops.sddmm_csr(ptr, idx, x1, g1, N), iters),
           E * (4 * 128 + 8) + 4 * N * 128 + 4 * E, 2 * E * 128)
    del x1, g1
    # per-node attention logits of the layer (both from one pass over x) and their gradients
    a_s, a_d = torch.randn(H, C, device="cuda"), torch.randn(H, C, device="cuda")
    gs = torch.randn(N, H, device="cuda")
    report("c3", "attention_logits fwd H=4 C=64 (src and dst logits)",
           timeit(lambda: _ops.attention_logits(x, a_s, a_d, N), iters), 4 * N * H * C + 8 * N * H, 4 * N * H * C)
    report("c3", "attention_logits bwd H=4 C=64 (grad x, grad att_src, grad att_dst)",
           timeit(lambda: _ops.attention_logits_bwd(x, a_s, a_d, gs, gs), iters), 8 * N * H * C + 8 * N * H,
           8 * N * H * C)
    # the same logits read off the layer's 128-column input (the layer's path when the input is
    # narrower than the transformed features): x @ m.T with m = att @ W per head
    xin, m = x.view(N, H * C)[:, :128].contiguous(), torch.randn(2 * H, 128, device="cuda")
    gxin = torch.zeros(N, 128, device="cuda")
    report("c3", "attention_logits from the 128-column input, fwd H=4",
           timeit(lambda: _ops.attention_logits_proj(xin, m, N, H), iters), 4 * N * 128 + 8 * N * H, 4 * N * 128 * H)
    report("c3", "attention_logits from the 128-column input, bwd H=4 (adds into grad x_in; grad m)",
           timeit(lambda: _ops.attention_logits_proj_bwd(xin, m, gs, gs, H, add_to=gxin), iters),
           12 * N * 128 + 8 * N * H, 8 * N * 128 * H)
    del x, g, gs, xin, gxin
    # the configuration's layer: GAT 128 -> 4 heads x 64, forward + backward through the
    # softmax and the edge-weighted aggregation including the edge-value gradient
    import cxgnncomp
    cxgnncomp.set_timers()
    layer = cxgnncomp.MyGATConv(128, 64, heads=4, concat=True).cuda()
    xin = torch.randn(N, 128, device="cuda").requires_grad_(True)
    gout = torch.randn(N, H * C, device="cuda") / 16

    def gat_step():
        xin.grad = None
        layer(xin, ptr, idx, N, N, E).backward(gout)
    report("c3", "MyGATConv 128 -> 4x64 fwd+bwd (linear, softmax, SpMM, SDDMM)", timeit(gat_step, max(2, iters // 3)))
    del layer, xin
    # one head, the reference's default (MyGATConv.forward_1): both orders of aggregation and transform
    for fin, fout in ((128, 256), (256, 256), (256, 64)):
        layer = cxgnncomp.MyGATConv(fin, fout, heads=1).cuda()
        xin = torch.randn(N, fin, device="cuda").requires_grad_(True)
        gout1 = torch.randn(N, fout, device="cuda") / 16

        def gat1_step():
            xin.grad = None
            layer(xin, ptr, idx, N, N, E).backward(gout1)
        report("c3", "MyGATConv one head %d -> %d fwd+bwd" % (fin, fout), timeit(gat1_step, max(2, iters // 3)))
        del layer, xin, gout1
    torch.cuda.empty_cache()
    # scheduling helpers (index work): bytes = arrays read + written once
    new_ptr, _ = cxgnncomp.neighbor_grouping(ptr, 32)
    n_groups = new_ptr.shape[0] - 1
    report("c3", "neighbor_grouping thres=32 (%d groups)" % n_groups,
           timeit(lambda: cxgnncomp.neighbor_grouping(ptr, 32), iters), 8 * (N + 1) * 2 + 16 * n_groups)
    eflag = torch.rand(E, device="cuda") < 0.5
    report("c3", "remove_from_graph_by_edge (half of the edges flagged)",
           timeit(lambda: cxgnncomp.remove_from_graph_by_edge(ptr, idx, eflag), iters),
           E * (1 + 8 + 8) + 8 * E // 2 + 8 * 3 * N)
    report("c3", "csr transpose (stable sort by source + fills)",
           timeit(lambda: _ops.csr_transpose(ptr, idx, N, N), max(2, iters // 4)), E * 8 * 4 + 16 * N)
    if CPU_BASELINE:
        from oracle import pyref
        cpu_spmm("c3", ptr, idx, N, 128, N // 8)
        rows = N // 16
        p, i = ptr[:rows + 1].cpu(), idx[:int(ptr[rows])].cpu()
        e = int(p[-1])
        a_s, a_d = att_s.cpu(), att_d.cpu()[:rows]
        cpu_report("c3", "edge_softmax_fwd H=4 op-wise torch",
                   lambda: pyref.edge_softmax_opwise(p, i, a_s, a_d, e, 0.2), "first %d rows, %d edges" % (rows, e),
                   e * (8 + 4 * H) + 5 * e * H + 4 * rows * H + 8 * (rows + 1))
        ne = 1 << 20
        xs, gs = torch.randn(N, H, C) / 8, torch.randn(rows, H, C) / 8
        d = torch.repeat_interleave(torch.arange(rows), p[1:] - p[:-1])[:ne]
        cpu_report("c3", "sddmm H=4 C=64 gathered einsum", lambda: pyref.sddmm_einsum(i[:ne], d, xs, gs),
                   "first %d edges" % ne, ne * (8 * H * C + 16) + 4 * ne * H)


def c4(iters):
    import cxgnncomp
    import cxgnncomp_backend as B
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _typed
    N, E, R, K = 1000000, 20000000, 16, 128
    ptr, idx, etype, _ = S.hetero_graph(N, E, num_rel=R, device="cuda")
    x = torch.randn(N, K, device="cuda") / 8
    w = torch.randn(R, K, K, device="cuda") * 0.02
    rel32 = etype.int()
    perm, seg = _typed.rel_segment(rel32, R)
    rows = B._ops.csr_row_ids(ptr, N, E)
    src, dst = idx[perm], rows[perm]
    out = torch.zeros(N, K, device="cuda")
    flops = 2.0 * E * K * K
    fused_bytes = E * (4 * K + 8 + 8 + 4 * K) + 4 * R * K * K
    report("c4", "rel_segment (stable sort by relation)", timeit(lambda: _typed.rel_segment(rel32, R), iters))
    layers = torch.tensor([N // 100, N // 10, N, N])
    report("c4", "rel_schedule (16 per-relation sub-graphs + layer table)",
           timeit(lambda: B.rel_schedule(ptr, idx, rel32, layers, R), max(2, iters // 4)))

    def fused(precision):
        out.zero_()
        _typed.typed_gemm(x, w, seg, E, src_idx=src, dst_idx=dst, out=out, atomic=True, precision=precision)
    report("c4", "rgcn fused gather-GEMM-scatter (fp32 atomics; not the layer's path) fp32 MFMA", timeit(lambda: fused("fp32"), iters), fused_bytes,
           flops, MFMA_F32)
    report("c4", "rgcn fused gather-GEMM-scatter (fp32 atomics; not the layer's path) fp32 as 6 bf16 products", timeit(lambda: fused("split6"), iters),
           fused_bytes, flops)
    report("c4", "rgcn fused gather-GEMM-scatter (fp32 atomics; not the layer's path) fp32 as 3 scaled fp16 products (default precision)",
           timeit(lambda: fused("split_f16"), iters), fused_bytes, flops)
    # the same result without atomics: one GEMM row per edge written in CSR order, then
    # the sum over each destination's consecutive rows (the sparse strategy of the layer)
    tmp = torch.empty(E, K, device="cuda")
    pos = torch.arange(E, device="cuda")

    def per_edge():
        _typed.typed_gemm(x, w, seg, E, src_idx=src, dst_idx=perm, out=tmp)
        B._ops.spmm(ptr, pos, tmp, N)
    report("c4", "rgcn gather-GEMM into per-edge rows + segment sum (no atomics), 3 scaled fp16 products",
           timeit(per_edge, iters), fused_bytes + 8 * E * K, flops)
    del tmp, pos
    x16 = x.to(torch.bfloat16)

    def fused16():
        out.zero_()
        _typed.typed_gemm(x16, w, seg, E, src_idx=src, dst_idx=dst, out=out, atomic=True, bf16=True)
    report("c4", "rgcn fused gather-GEMM-scatter (fp32 atomics; not the layer's path) bf16 MFMA", timeit(fused16, iters),
           E * (2 * K + 16 + 4 * K) + 2 * R * K * K, flops, MFMA_BF16)
    xe = torch.empty(E, K, device="cuda")
    xe.normal_()
    oe = torch.empty(E, K, device="cuda")
    report("c4", "typed GEMM edge->edge fp32 (E x 128 x 128, sorted rows)",
           timeit(lambda: _typed.typed_gemm(xe, w, seg, E, out=oe, precision="fp32"), iters),
           E * 8 * K + 4 * R * K * K, flops, MFMA_F32)
    report("c4", "typed GEMM edge->edge fp32 as 3 scaled fp16 products (default precision)",
           timeit(lambda: _typed.typed_gemm(xe, w, seg, E, out=oe, precision="split_f16"), iters),
           E * 8 * K + 4 * R * K * K, flops)
    for prec, nprod in (("split6", 6), ("split3", 3)):
        report("c4", "typed GEMM edge->edge fp32 as %d bf16 products" % nprod,
               timeit(lambda: _typed.typed_gemm(xe, w, seg, E, out=oe, precision=prec), iters),
               E * 8 * K + 4 * R * K * K, flops)
    xe16 = xe.to(torch.bfloat16)
    report("c4", "typed GEMM edge->edge bf16",
           timeit(lambda: _typed.typed_gemm(xe16, w, seg, E, out=oe, bf16=True), iters),
           E * 6 * K + 2 * R * K * K, flops, MFMA_BF16)
    del xe, oe, xe16
    # the hidden-256 shape of a deeper relational model: 5M rows x 256 x 256
    E2, K2 = 5000000, 256
    x2 = torch.randn(E2, K2, device="cuda") / 8
    w2 = torch.randn(R, K2, K2, device="cuda") * 0.02
    seg2 = (seg.double() * (E2 / E)).long()
    seg2[-1] = E2
    o2 = torch.empty(E2, K2, device="cuda")
    for prec, what in (("fp32", "fp32 MFMA"), ("split_f16", "3 scaled fp16 products (default precision; the tiled kernel for wide operands)")):
        report("c4", "typed GEMM 5M rows x 256 x 256, %s" % what,
               timeit(lambda: _typed.typed_gemm(x2, w2, seg2, E2, out=o2, precision=prec), iters),
               E2 * 8 * K2 + 4 * R * K2 * K2, 2.0 * E2 * K2 * K2, MFMA_F32 if prec == "fp32" else None)
    del x2, w2, o2
    global _last_spread
    t_mm = (E / N) * timeit(lambda: torch.mm(x, w[0]), iters)
    _last_spread = tuple((E / N) * v for v in _last_spread)
    report("c4", "torch.mm [1M,128]x[128,128] x 20 (library GEMM of the same flops, no gather, for scale)",
           t_mm, E * 8 * K, flops, MFMA_F32)
    # the remaining relational entry points
    xr = torch.randn(R * (N // R), K, device="cuda") / 8         # [R * nodes, F] pre-transformed features
    nodes_r = N // R
    idx_r = idx % nodes_r
    report("c4", "aggr_rel forward (relation-offset gather) F=128",
           timeit(lambda: B.aggr_rel(xr, ptr, idx_r, rel32, N, R), iters), spmm_bytes(N, E, K) + 4 * E, E * K)
    xrg = xr.clone().requires_grad_(True)
    gn = torch.randn(N, K, device="cuda") / 16

    def aggr_rel_step():
        xrg.grad = None
        B.aggr_rel(xrg, ptr, idx_r, rel32, N, R).backward(gn)
    report("c4", "aggr_rel forward + backward (gather over the transposed combined index) F=128", timeit(aggr_rel_step, iters))
    del xr, xrg
    oe2 = torch.zeros(E, K, device="cuda")
    report("c4", "typed_linear_s2e (out[e] += x[src[e]] W[type[e]]), 3 scaled fp16 products",
           timeit(lambda: B.typed_linear_s2e(x, w, oe2, idx, rel32), max(2, iters // 2)),
           E * (4 * K + 8 * K + 12) + 4 * R * K * K, flops)
    del oe2
    on = torch.zeros(N, K, device="cuda")
    report("c4", "typed_linear_s2d (out[dst[e]] += x[src[e]] W[type[e]]; products of the (source, type) pairs that occur, summed per destination)",
           timeit(lambda: B.typed_linear_s2d(x, w, on, idx, rows, rel32), max(2, iters // 2)),
           fused_bytes, flops)
    del on
    from cxgnncomp.typed_linear import TypedLinearE2EOP
    xeg = torch.randn(E, K, device="cuda").requires_grad_(True)
    wg = w.clone().requires_grad_(True)
    pre = TypedLinearE2EOP.preprocess(w, etype)
    ge = torch.randn(E, K, device="cuda") / 16

    def e2e_step():
        xeg.grad = None
        wg.grad = None
        TypedLinearE2EOP.apply(xeg, wg, etype, pre).backward(ge)
    report("c4", "TypedLinearE2EOP forward + backward (edge-level x, preprocessed)", timeit(e2e_step, max(2, iters // 3)))
    del xeg, ge, pre
    from cxgnncomp.typed_linear import (TypedLinearS2DAggrMMOP, TypedLinearS2DMMAggrOP, TypedLinearS2DSort,
                                        TypedLinearS2EOP)
    pre_s2e = TypedLinearS2EOP.preprocess(w, etype, idx, 256)
    report("c4", "TypedLinearS2EOP forward (node-level x gathered per edge, preprocessed)",
           timeit(lambda: TypedLinearS2EOP.apply(x, w, etype, idx, pre_s2e), max(2, iters // 3)),
           E * (4 * K + 4 * K + 16) + 4 * R * K * K, flops)
    del pre_s2e
    xr1 = x.clone().requires_grad_(True)
    wr1 = w.clone().requires_grad_(True)

    def op_step(op):
        def run():
            xr1.grad = None
            wr1.grad = None
            op(xr1, wr1, ptr, idx, etype, N).backward(gn)
        return run
    report("c4", "RGCNOP = TypedLinearS2DMMAggrOP fwd+bwd (transform all nodes for all relations, then aggregate)",
           timeit(op_step(TypedLinearS2DMMAggrOP.apply), max(2, iters // 3)))
    report("c4", "RGCNOP2 = TypedLinearS2DAggrMMOP fwd+bwd (aggregate per (destination, relation), then transform)",
           timeit(op_step(TypedLinearS2DAggrMMOP.apply), max(2, iters // 3)))
    report("c4", "TypedLinearS2DSort fwd+bwd (relation-segmented edges, one typed GEMM)",
           timeit(op_step(TypedLinearS2DSort), 2))
    from cxgnncomp import graph_conv as _gc
    report("c4", "RGCNOP (by its upstream name; CUDA tensors take TypedLinearS2DMMAggrOP) fwd+bwd",
           timeit(op_step(_gc.RGCNOP.apply), max(2, iters // 3)))
    report("c4", "RGCNOP3 = aggr_rgcn_direct_func with its gradients, fwd+bwd",
           timeit(op_step(_gc.RGCNOP3.apply), max(2, iters // 3)))
    report("c4", "SeastarRGCNOP = seastar_forward + seastar_backward, fwd+bwd",
           timeit(op_step(_gc.SeastarRGCNOP.apply), max(2, iters // 3)))
    del xr1, wr1
    layer = cxgnncomp.MyRGCNConv(K, K, R).cuda()
    xg = x.clone().requires_grad_(True)

    gout = torch.randn(N, K, device="cuda") / 16

    def layer_step():
        xg.grad = None
        layer(xg, ptr, idx, etype, N).backward(gout)
    report("c4", "MyRGCNConv layer fwd+bwd (typed transform, relational aggregate, /deg)",
           timeit(layer_step, max(2, iters // 3)))
    layer16 = cxgnncomp.MyRGCNConv(K, K, R, precision="bf16").cuda()

    def layer16_step():
        xg.grad = None
        layer16(xg, ptr, idx, etype, N).backward(gout)
    report("c4", "MyRGCNConv layer fwd+bwd, bf16 variant (bf16 operands of the forward and input-gradient GEMMs, pair-row tables kept in bf16, fp32 accumulation)",
           timeit(layer16_step, max(2, iters // 3)))
    if CPU_BASELINE:
        from oracle import pyref
        rows = N // 32
        p, i, t = ptr[:rows + 1].cpu(), idx[:int(ptr[rows])].cpu(), etype[:int(ptr[rows])].cpu()
        xc, wc = x.cpu(), w.cpu()
        cpu_report("c4", "rgcn forward, relation-sorted torch (TypedLinearS2DSort)",
                   lambda: pyref.typed_linear_s2d_sort(xc, wc, p, i, t, rows),
                   "first %d rows, %d edges" % (rows, int(p[-1])))


def c5(iters):
    import cxgnncomp
    from cxgnncomp import synthetic as S
    ptr, idx, nn, ne = S.sampled_batch(device="cuda")
    n_src = nn[-1]
    x = torch.randn(n_src, 128, device="cuda")
    layers = [cxgnncomp.MySageConv(128, 256).cuda(), cxgnncomp.MySageConv(256, 256).cuda(),
              cxgnncomp.MySageConv(256, 47).cuda()]
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _ops
    if C5_STEPS > 0:
        # only the training step, C5_STEPS times: for kernel traces that count launches per batch
        # (trace N and 2N steps and take the difference) and for the host's share of a step
        import time
        xg = x.clone().requires_grad_(True)
        gout = torch.randn(nn[0], 47, device="cuda")

        def one_step():
            if C5_FRESH:
                _ops.clear_graph_cache()        # a new sampled batch: nothing of the graph is cached
                _ops.note_edge_counts(ptr, idx, nn[:3], ne)   # ... but its layer sizes are known (as GNN.forward_cxg does)
            xg.grad = None
            h = xg
            for li, layer in enumerate(layers):
                h = layer(h, ptr, idx, nn[2 - li])
                if li < 2:
                    h = torch.relu(h)
            h.backward(gout)
        for _ in range(3):
            one_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(C5_STEPS):
            one_step()
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        print(json.dumps({"config": "c5", "op": "3-layer SAGE fwd+bwd, %d steps after 3 warm-up steps, %s"
                          % (C5_STEPS, "graph cache cleared before every step" if C5_FRESH else "reversed graphs cached"),
                          "host_enqueue_ms_per_step": round((t1 - t0) * 1e3 / C5_STEPS, 4),
                          "wall_ms_per_step": round((t2 - t0) * 1e3 / C5_STEPS, 4)}), flush=True)
        return
    for li, (rows, edges) in enumerate(zip(nn[2::-1], ne[::-1])):
        report("c5", "sage_mean_forward rows=%d edges=%d F=128" % (rows, edges),
               timeit(lambda: B.sage_mean_forward(x, ptr, idx, rows), iters), spmm_bytes(rows, edges, 128), edges * 128)

    def prepare_sorts():
        # the reversed graph of each layer by its own stable sort
        for li, rows in enumerate(nn[2::-1]):
            _ops.csr_transpose(ptr, idx, rows, nn[3 - li])

    def prepare():
        # what a NEW batch pays once before its first backward: the reversed graph of the largest
        # layer by a stable sort, the two smaller ones cut out of it (they are edge prefixes)
        _ops.clear_graph_cache()
        for li, rows in enumerate(nn[2::-1]):
            _ops.note_layer(ptr, idx, rows, nn[3 - li])
        for li, rows in enumerate(nn[:3]):
            _ops.transposed(ptr, idx, rows, nn[li + 1])
    report("c5", "per-batch preparation, three stable sorts: reversed CSR of the 3 layers", timeit(prepare_sorts, iters))
    report("c5", "per-batch preparation: reversed CSR of the largest layer (stable sort + fills), the two smaller "
                 "ones compacted out of it", timeit(prepare, iters))
    xg = x.clone().requires_grad_(True)
    gout_b = torch.randn(nn[0], 47, device="cuda") / 16    # the gradient a loss would hand back

    x_frozen = x.clone()                     # input features that need no gradient: the normal training case

    def frozen_batch_step():
        _ops.clear_graph_cache()
        _ops.note_edge_counts(ptr, idx, nn[:3], ne)
        h = x_frozen
        for li, layer in enumerate(layers):
            h = layer(h, ptr, idx, nn[2 - li])
            if li < 2:
                h = torch.relu(h)
        h.backward(gout_b)

    def batch_step():
        xg.grad = None
        h = xg
        for li, layer in enumerate(layers):
            h = layer(h, ptr, idx, nn[2 - li])
            if li < 2:
                h = torch.relu(h)
        h.backward(gout_b)
    launches = "kernel launches per batch counted with rocprofv3 kernel traces of 10 and 20 steps"
    report("c5", "3-layer SAGE fwd+bwd per batch, reversed graphs cached (%s nodes per layer)" % nn,
           timeit(batch_step, iters), note=launches)

    def new_batch_step():
        _ops.clear_graph_cache()                 # a new sampled batch: nothing of the graph is cached
        _ops.note_edge_counts(ptr, idx, nn[:3], ne)   # ... but its layer sizes are known (as GNN.forward_cxg does)
        batch_step()
    report("c5", "3-layer SAGE fwd+bwd per NEW batch, preparation of the reversed graphs included",
           timeit(new_batch_step, iters), note=launches)
    report("c5", "3-layer SAGE fwd+bwd per NEW batch, input features without gradient (the first layer needs no reversed graph)",
           timeit(frozen_batch_step, iters), note=launches)
    if CPU_BASELINE:
        cpu_spmm("c5", ptr, idx, n_src, 128, nn[2])


def e3(iters):
    """The one typed-linear shape the reference stores timings for (test/ae/E3_ablation/test-batch.py:27-52,
    output kept in process-batch-data.ipynb): the 169,343-node / 2,332,486-edge citation graph, 512 -> 512,
    7 random relations; source -> edge typed linear.  The reference's stored numbers, hardware unstated:
    Triton typed_matmul 18.76 - 27.92 ms, per-edge kernel typed_linear_s2e 417.36 ms."""
    import cxgnncomp as cxgc
    import cxgnncomp_backend as B
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _typed
    ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, seed=0, device="cuda")
    n, E, K, R = ptr.shape[0] - 1, idx.shape[0], 512, 7
    torch.manual_seed(0)
    x = torch.randn(n, K, device="cuda")
    rel = torch.randint(0, R, (E,), dtype=torch.int32, device="cuda")
    rel64 = rel.long()
    w = torch.randn(R, K, K, device="cuda")
    flops = 2.0 * E * K * K
    nbytes = E * (4 * K + 4 * K + 8) + 4 * R * K * K
    pre = cxgc.TypedLinearS2EOP.preprocess(w, rel64, idx, thres=256)
    report("e3", "TypedLinearS2EOP forward (typed_matmul, source -> edge), E=2,332,486 K=N=512 R=7",
           timeit(lambda: cxgc.TypedLinearS2EOP.apply(x, w, rel64, idx, pre), iters), nbytes, flops,
           note="reference's stored Triton typed_matmul: 18.76-27.92 ms (hardware unstated)")
    out = torch.zeros(E, K, device="cuda")
    report("e3", "typed_linear_s2e (accumulates into the caller's rows)",
           timeit(lambda: B.typed_linear_s2e(x, w, out, idx, rel, 32), iters), nbytes + 4 * E * K, flops,
           note="reference's stored per-edge kernel: 417.36 ms (hardware unstated)")
    del out
    perm, seg = _typed.rel_segment(rel, R)
    xe = torch.randn(E, K, device="cuda")
    oe = torch.empty(E, K, device="cuda")
    report("e3", "typed GEMM over relation-sorted rows, plain (E x 512 x 512), 3 scaled fp16 products",
           timeit(lambda: _typed.typed_gemm(xe, w, seg, E, out=oe, precision="split_f16"), iters), nbytes, flops)
    report("e3", "same, fp32 MFMA",
           timeit(lambda: _typed.typed_gemm(xe, w, seg, E, out=oe, precision="fp32"), iters), nbytes, flops, MFMA_F32)
    src = idx[perm].contiguous()
    report("e3", "typed GEMM with gathered source rows, relation-sorted output",
           timeit(lambda: _typed.typed_gemm(x, w, seg, E, src_idx=src, out=oe, precision="split_f16"), iters),
           nbytes, flops)
    g = torch.randn(E, K, device="cuda")
    report("e3", "weight gradient over the edge rows (gathered sources), [7, 512, 512]",
           timeit(lambda: _typed.typed_gemm_wgrad(x, g, seg, E, R, src_idx=src), iters), nbytes, flops)
    global _last_spread
    t_mm = timeit(lambda: torch.mm(xe, w[0], out=oe), iters)
    report("e3", "torch.mm [E,512]x[512,512] (library fp32 GEMM of the same flops, one relation, for scale)",
           t_mm, nbytes, flops, MFMA_F32)
    xg = x.clone().requires_grad_(True)
    wg = w.clone().requires_grad_(True)

    def step():
        xg.grad = wg.grad = None
        cxgc.TypedLinearS2EOP.apply(xg, wg, rel64, idx, pre).backward(g)
    report("e3", "TypedLinearS2EOP forward + backward (grad x and grad W)", timeit(step, iters), 3 * nbytes, 3 * flops)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--configs", default="c1,c2,c3,c4,c5")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--cold", action="store_true", help="flush the caches before every timed call")
    ap.add_argument("--cpu-baseline", action="store_true", help="also time the host-side PyTorch restatements")
    ap.add_argument("--c5-steps", type=int, default=0,
                    help="c5 only: run just the 3-layer SAGE training step this many times (for launch counting)")
    ap.add_argument("--c5-fresh", action="store_true", help="with --c5-steps: clear the graph cache before every step")
    args = ap.parse_args()
    global COLD, CPU_BASELINE, C5_STEPS, C5_FRESH
    COLD, CPU_BASELINE, C5_STEPS, C5_FRESH = args.cold, args.cpu_baseline, args.c5_steps, args.c5_fresh
    sys.path.insert(0, os.path.dirname(HERE))
    table = {"c1": c1, "c2": c2, "c3": c3, "c4": c4, "c5": c5, "e3": e3}
    for name in args.configs.split(","):
        table[name](args.iters)
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
