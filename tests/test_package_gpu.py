"""The cxgnncomp Python surface (autograd ops, typed_linear family, conv layers,
alternative-implementation names) on the GPU against CPU restatements."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close
from oracle import pyref
from test_spmm_gpu import ATOL, RTOL, _graph, _scale

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _hetero(n=2000, e=30000, R=5, seed=6):
    from cxgnncomp import synthetic as S
    ptr, idx, etype, _ = S.hetero_graph(n, e, num_rel=R, seed=seed)
    return ptr, idx, etype


def _rgcn_reference(x, w, ptr, idx, rel, n, g):
    """Forward and gradients of sum_e x[idx[e]] @ W[rel[e]] by autograd through the
    reference's pure-torch relation-sorted form, in float64 on the CPU."""
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    out = pyref.typed_linear_s2d_sort(x64, w64, ptr, idx, rel, n)
    out.backward(g.double())
    return out.detach().numpy(), x64.grad.numpy(), w64.grad.numpy()


@pytest.mark.parametrize("opname", ["AggrOP", "AggrDirectedOP"])
def test_aggr_ops_true_transposed_backward(opname):
    import cxgnncomp
    from cxgnncomp import graph_conv
    from cxgnncomp import synthetic as S
    op = getattr(graph_conv, opname)
    # bipartite, non-symmetric: 900 destinations, 1500 sources
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=900, fanouts=(6,), id_space=1400, seed=3)
    n_dst, n_src = nn[0], nn[1]
    torch.manual_seed(15)
    x = (torch.randn(n_src, 64) / 3).cuda().requires_grad_(True)
    g = torch.randn(n_dst, 64) / 3
    announce("%s fwd+bwd" % opname)
    out = op.apply(x, ptr.cuda(), idx.cuda(), torch.tensor(n_dst))
    out.backward(g.cuda())
    torch.cuda.synchronize()
    assert_close(_np(out), oracle.spmm(ptr.numpy(), idx.numpy(), _np(x), n_dst), RTOL, ATOL, "fwd")
    assert_close(_np(x.grad), oracle.spmm_bwd(ptr.numpy(), idx.numpy(), g.numpy(), n_dst, n_src), RTOL, ATOL, "bwd")
    assert "run_spmm_configurable_lazy" in cxgnncomp.global_tuner.cache


def test_spmm_val_op():
    from cxgnncomp.graph_kernel import SpMMValOP
    ptr, idx = _graph("powerlaw")
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    H, C = 4, 64
    torch.manual_seed(16)
    sc = _scale(ptr)
    x = (torch.randn(n, H, C) * sc).cuda().requires_grad_(True)
    val = torch.rand(E, H).cuda().requires_grad_(True)
    g = torch.randn(n, H, C) * sc
    announce("SpMMValOP H=4 C=64")
    out = SpMMValOP.apply(x, ptr.cuda(), idx.cuda(), val, n)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    p, i = ptr.numpy(), idx.numpy()
    assert_close(_np(out), oracle.spmm(p, i, _np(x), n, val=_np(val)), RTOL, ATOL, "fwd")
    assert_close(_np(x.grad), oracle.spmm_bwd(p, i, g.numpy(), n, n, val=_np(val)), RTOL, ATOL, "grad x")
    assert_close(_np(val.grad), oracle.edge_grad(p, i, _np(x), g.numpy(), n), RTOL, ATOL, "grad val (per head)")


def test_typed_matmul_index_modes():
    import cxgnncomp
    torch.manual_seed(17)
    M, K, N, R = 700, 64, 48, 4
    a = torch.randn(M, K) / 8
    b = torch.randn(R, K, N)
    rel = torch.sort(torch.randint(0, R, (M,)))[0]
    src = torch.randint(0, M, (M,))
    dst = torch.randperm(M)
    ac, bc, rc = a.cuda(), b.cuda(), rel.cuda()
    announce("typed_matmul no index")
    c = cxgnncomp.typed_matmul(ac, bc, rc)
    ref = pyref.typed_matmul(a.double(), b.double(), rel).numpy()
    assert_close(_np(c), ref, RTOL, ATOL, "no index")
    announce("typed_matmul seq_output")
    c = cxgnncomp.typed_matmul(ac, bc, rc, M, src.cuda(), seq_output=True)
    ref = pyref.typed_matmul(a.double(), b.double(), rel, src).numpy()
    assert_close(_np(c), ref, RTOL, ATOL, "seq output")
    announce("typed_matmul double index")
    c = cxgnncomp.typed_matmul(ac, bc, rc, M, src.cuda(), dst.cuda())
    assert_close(_np(c), pyref.typed_matmul(a.double(), b.double(), rel, src, dst).numpy(), RTOL, ATOL, "double")
    announce("typed_matmul single index (permutation with padding)")
    perm = torch.randperm(M)
    padded = torch.cat([perm, torch.full((9,), -1)])
    relp = torch.cat([rel, torch.full((9,), R)])
    c = cxgnncomp.typed_matmul(ac, bc, relp.cuda(), M, padded.cuda())
    want = torch.zeros(M, N, dtype=torch.float64)
    want[perm] = torch.bmm(a[perm].double().unsqueeze(1), b[rel].double()).squeeze(1)
    assert_close(_np(c), want.numpy(), RTOL, ATOL, "single index")
    announce("typed_matmul unsorted rel")
    rel_u = torch.randint(0, R, (M,))
    c = cxgnncomp.typed_matmul(ac, bc, rel_u.cuda())
    assert_close(_np(c), pyref.typed_matmul(a.double(), b.double(), rel_u).numpy(), RTOL, ATOL, "unsorted")


def test_typed_linear_e2e_and_s2e_ops():
    import cxgnncomp
    torch.manual_seed(18)
    E, K, N, R, n_src = 3000, 64, 32, 5, 400
    types = torch.randint(0, R - 1, (E,))                 # highest relation absent
    w = torch.randn(R, K, N) / 4
    x = torch.randn(E, K) / 8
    g = torch.randn(E, N)
    pre = cxgnncomp.TypedLinearE2EOP.preprocess(w.cuda(), types.cuda(), 32)
    sorted_types, num_item, indices, count = pre
    assert num_item == E and count.device.type == "cpu" and count.tolist() == torch.bincount(types, minlength=R).tolist()
    st, _, ind, _ = pyref.e2e_preprocess(R, types.numpy(), 32)
    assert np.array_equal(_np(sorted_types), st) and np.array_equal(_np(indices), ind)
    xg = x.cuda().requires_grad_(True)
    wg = w.cuda().requires_grad_(True)
    announce("TypedLinearE2EOP fwd+bwd")
    out = cxgnncomp.TypedLinearE2EOP.apply(xg, wg, types.cuda(), pre)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
    ref = torch.bmm(x64.unsqueeze(1), w64[types]).squeeze(1)
    ref.backward(g.double())
    assert out.shape == (E, N)
    assert_close(_np(out), ref.detach().numpy(), RTOL, ATOL, "e2e fwd")
    assert_close(_np(xg.grad), x64.grad.numpy(), RTOL, 2 * ATOL, "e2e grad x")
    sc = float(w64.grad.abs().max())
    assert_close(_np(wg.grad) / sc, w64.grad.numpy() / sc, RTOL, ATOL, "e2e grad w")
    # without a preprocessed list the op prepares itself
    out2 = cxgnncomp.TypedLinearE2EOP.apply(x.cuda(), w.cuda(), types.cuda())
    assert torch.equal(out2, out.detach())
    # source -> edge
    xs = torch.randn(n_src, K) / 8
    src = torch.randint(0, n_src, (E,))
    xsg = xs.cuda().requires_grad_(True)
    wg2 = w.cuda().requires_grad_(True)
    announce("TypedLinearS2EOP fwd+bwd")
    out = cxgnncomp.TypedLinearS2EOP.apply(xsg, wg2, types.cuda(), src.cuda(), [], 32)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    xs64, w64 = xs.double().requires_grad_(True), w.double().requires_grad_(True)
    ref = torch.bmm(xs64[src].unsqueeze(1), w64[types]).squeeze(1)
    ref.backward(g.double())
    assert_close(_np(out), ref.detach().numpy(), RTOL, ATOL, "s2e fwd")
    sx = float(xs64.grad.abs().max())
    assert_close(_np(xsg.grad) / sx, xs64.grad.numpy() / sx, RTOL, ATOL, "s2e grad x")
    assert_close(_np(wg2.grad) / sc, w64.grad.numpy() / sc, RTOL, 2 * ATOL, "s2e grad w")


@pytest.mark.parametrize("tables", ["dense", "pairs"])
@pytest.mark.parametrize("opname", ["RGCNOP", "RGCNOP2", "RGCNOP3", "SeastarRGCNOP",
                                    "TypedLinearS2DMMAggrOP", "TypedLinearS2DAggrMMOP"])
def test_rgcn_op_variants(opname, tables, monkeypatch):
    """Every RGCN operator name, with the intermediate tables holding a row for every (node,
    relation) pair and with a row only for the pairs that own an edge."""
    import cxgnncomp
    from cxgnncomp import graph_conv
    from cxgnncomp_backend import _typed
    monkeypatch.setattr(_typed, "RGCN_PAIR_FILL_MAX", 2.0 if tables == "pairs" else -1.0)
    cxgnncomp.set_timers()
    ptr, idx, etype = _hetero()
    n = ptr.shape[0] - 1
    K, N, R = 64, 32, 5
    torch.manual_seed(19)
    x = torch.randn(n, K) / 16
    w = torch.randn(R, K, N) / 2
    g = torch.randn(n, N) / 4
    want, want_gx, want_gw = _rgcn_reference(x, w, ptr, idx, etype, n, g)
    op = getattr(graph_conv, opname, None) or getattr(cxgnncomp, opname)
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    announce("%s fwd+bwd" % opname)
    out = op.apply(xg, wg, ptr.cuda(), idx.cuda(), etype.cuda(), n)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    assert_close(_np(out), want, RTOL, 2 * ATOL, opname + " fwd")
    assert_close(_np(xg.grad), want_gx, RTOL, 2 * ATOL, opname + " grad x")
    sc = float(np.abs(want_gw).max())
    assert_close(_np(wg.grad) / sc, want_gw / sc, RTOL, 2 * ATOL, opname + " grad w")


def test_rgcn_sorted_variant_on_gpu():
    """TypedLinearS2DSort with GPU tensors: same values and gradients as the torch composition
    of the reference (restated in oracle/pyref.py) in double precision."""
    import cxgnncomp
    ptr, idx, etype = _hetero()
    n = ptr.shape[0] - 1
    K, N, R = 64, 32, 5
    torch.manual_seed(23)
    x = torch.randn(n, K) / 16
    w = torch.randn(R, K, N) / 2
    g = torch.randn(n, N) / 4
    want, want_gx, want_gw = _rgcn_reference(x, w, ptr, idx, etype, n, g)
    for fn in (cxgnncomp.TypedLinearS2DSort,):
        xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
        announce("%s on GPU tensors" % fn.__name__)
        out = fn(xg, wg, ptr.cuda(), idx.cuda(), etype.cuda(), n)
        out.backward(g.cuda())
        torch.cuda.synchronize()
        assert_close(_np(out), want, RTOL, 2 * ATOL, "sorted fwd")
        assert_close(_np(xg.grad), want_gx, RTOL, 2 * ATOL, "sorted grad x")
        sc = float(np.abs(want_gw).max())
        assert_close(_np(wg.grad) / sc, want_gw / sc, RTOL, 2 * ATOL, "sorted grad w")


def test_rgcn_named_variants_and_prune_path():
    import cxgnncomp
    import cxgnncomp_backend as B
    ptr, idx, etype = _hetero()
    n = ptr.shape[0] - 1
    K, N, R = 64, 32, 5
    torch.manual_seed(20)
    x = torch.randn(n, K) / 16
    w = torch.randn(R, K, N) / 2
    want = oracle.rgcn_fused(x.numpy(), ptr.numpy(), idx.numpy(), w.numpy(), etype.numpy(), n)
    pc, ic, ec, xc, wc = ptr.cuda(), idx.cuda(), etype.cuda(), x.cuda(), w.cuda()
    for name in ("rgcn_triton", "rgcn_triton_opt", "rgcn_scatter"):
        announce(name)
        assert_close(_np(getattr(cxgnncomp, name)(xc, pc, ic, ec, wc, n)), want, RTOL, 2 * ATOL, name)
    for name in ("rgcn_full_mm", "rgcn_full_mm2"):
        announce(name)
        assert_close(_np(getattr(cxgnncomp, name)(xc, pc, ic, ec, wc, n, R)), want, RTOL, 2 * ATOL, name)
    announce("rel_schedule on GPU tensors + rgcn_prune_mm")
    meta = B.rel_schedule(pc, ic, ec.int(), torch.tensor([n, n]), R)
    want_meta = oracle.rel_schedule(ptr.numpy(), idx.numpy(), etype.numpy(), [n, n], R)
    for gmeta, wmeta in zip(meta, want_meta):
        assert np.array_equal(_np(gmeta), wmeta)
    assert_close(_np(cxgnncomp.rgcn_prune_mm(xc, wc, meta, n, R)), want, RTOL, 2 * ATOL, "prune mm")
    announce("rgcn_just_aggr / rgcn_just_aggr_prune")
    agg = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n)
    wk = torch.zeros(R, K, K)
    assert_close(_np(cxgnncomp.rgcn_just_aggr(xc, pc, ic, ec, wk.cuda(), n, R)), agg, RTOL, ATOL, "just aggr")
    assert_close(_np(cxgnncomp.rgcn_just_aggr_prune(xc, meta, n, R)), agg, RTOL, ATOL, "just aggr prune")
    announce("TypedLinearS2DPushOP")
    dst = torch.repeat_interleave(torch.arange(n), ptr[1:] - ptr[:-1])
    got = cxgnncomp.TypedLinearS2DPushOP(xc, wc, ec, ic, dst.cuda(), R, n, idx.shape[0])
    assert_close(_np(got), want, RTOL, 2 * ATOL, "push op")


def test_rgcn_full_bmm_and_run_rgcn4():
    """rgcn_full_bmm (basis decomposition W_rel = sum_b comp[rel, b] basis[b],
    cxgnncomp/codegen/rgcn_kernel.py:445-461) against the fused oracle on the composed weights,
    and run_rgcn4 (gather, edge-level typed linear, per-destination sum, graph_conv.py:309-326),
    forward and both gradients, against the float64 restatement."""
    import cxgnncomp
    from cxgnncomp.graph_conv import run_rgcn4
    from cxgnncomp.typed_linear import TypedLinearE2EOP
    from oracle import pyref
    ptr, idx, etype = _hetero()
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    K, N, R, Bs = 64, 32, 5, 3
    torch.manual_seed(23)
    x = torch.randn(n, K) / 16
    basis = torch.randn(Bs, K, N) / 2
    comp = torch.randn(R, Bs)
    w_full = torch.einsum("rb,bio->rio", comp, basis)
    want = oracle.rgcn_fused(x.numpy(), ptr.numpy(), idx.numpy(), w_full.numpy(), etype.numpy(), n)
    announce("rgcn_full_bmm")
    got = cxgnncomp.rgcn_full_bmm(x.cuda(), ptr.cuda(), idx.cuda(), etype.cuda(), basis.cuda(), comp.cuda(), n, R)
    assert_close(_np(got), want, RTOL, 2 * ATOL, "rgcn_full_bmm")
    # run_rgcn4
    w = torch.randn(R, K, N) / 2
    g = torch.randn(n, N) / 4
    x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
    o64 = pyref.typed_linear_s2d_sort(x64, w64, ptr, idx, etype, n)
    o64.backward(g.double())
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    et = etype.cuda()
    announce("run_rgcn4 fwd+bwd")
    pre = TypedLinearE2EOP.preprocess(wg.detach(), et)
    out = run_rgcn4(xg, ptr.cuda(), idx.cuda(), et, wg, n, E, pre)
    out.backward(g.cuda())
    assert_close(_np(out), o64.detach().numpy(), RTOL, 2 * ATOL, "run_rgcn4 forward")
    scx = max(1.0, float(x64.grad.abs().max()))
    assert_close(_np(xg.grad) / scx, x64.grad.numpy() / scx, RTOL, 2 * ATOL, "run_rgcn4 grad x")
    scw = float(w64.grad.abs().max())
    assert_close(_np(wg.grad) / scw, w64.grad.numpy() / scw, RTOL, 2 * ATOL, "run_rgcn4 grad w")


def test_alternative_spmm_sddmm_names_and_prof():
    import cxgnncomp
    ptr, idx = _graph("uniform")
    n = ptr.shape[0] - 1
    torch.manual_seed(21)
    x = torch.randn(n, 64) / 4
    val = torch.rand(idx.shape[0])
    pc, ic, xc = ptr.cuda(), idx.cuda(), x.cuda()
    announce("spmm_triton / spmm_torch / spmm_mm_triton")
    a = cxgnncomp.spmm_triton(xc, pc, ic, n)
    b = cxgnncomp.spmm_torch(xc, pc, ic, n)
    assert_close(_np(a), _np(b), 1e-4, 1e-5, "hip vs torch.sparse.mm on the GPU")
    a = cxgnncomp.spmm_triton(xc, pc, ic, n, val.cuda())
    assert_close(_np(a), oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n, val=val.numpy()), RTOL, ATOL, "val")
    w = torch.randn(16, 64) / 8
    got = cxgnncomp.spmm_mm_triton(xc, pc, ic, w.cuda(), n)
    want = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n).astype(np.float64) @ w.numpy().T
    assert_close(_np(got), want, 1e-4, 1e-4, "spmm+mm")
    announce("sddmm_dense")
    dst = torch.repeat_interleave(torch.arange(n), ptr[1:] - ptr[:-1])
    srcf = torch.randn(n, 64, 4) / 8                       # [num_src, feat, head]
    got = cxgnncomp.sddmm_dense(xc, srcf.cuda(), dst.cuda(), ic, idx.shape[0])
    want = np.einsum("ek,ekh->eh", x.numpy()[dst.numpy()].astype(np.float64), srcf.numpy()[idx.numpy()])
    assert_close(_np(got), want, RTOL, ATOL, "sddmm_dense")
    res = cxgnncomp.prof("spmm", "hip", lambda: cxgnncomp.spmm_triton(xc, pc, ic, n), display=False)
    assert len(res) == 3 and res[1] <= res[0] <= res[2] and cxgnncomp.global_res[-1] == res


def test_conv_layers_forward_backward():
    """Layers against the same layer evaluated on the CPU with dense torch ops."""
    import cxgnncomp
    cxgnncomp.set_timers()
    ptr, idx = _graph("powerlaw")
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    p, i = ptr.numpy(), idx.numpy()
    dst = torch.repeat_interleave(torch.arange(n), ptr[1:] - ptr[:-1])
    deg = (ptr[1:] - ptr[:-1]).double()
    torch.manual_seed(22)
    x = torch.randn(n, 32) / 20
    pc, ic = ptr.cuda(), idx.cuda()

    def agg(t, weight=None):
        msg = t[idx] if weight is None else t[idx] * weight.reshape(E, *([1] * (t.dim() - 1)))
        return torch.zeros((n,) + tuple(t.shape[1:]), dtype=t.dtype).index_add_(0, dst, msg)

    def check(layer, ref_fn, args, name):
        xg = x.cuda().requires_grad_(True)
        layer = layer.cuda()
        announce(name)
        out = layer(xg, *args)
        out.sum().backward()
        torch.cuda.synchronize()
        x64 = x.double().requires_grad_(True)
        params = {k: v.detach().double().cpu().requires_grad_(True) for k, v in layer.named_parameters()}
        ref = ref_fn(x64, params)
        ref.sum().backward()
        assert_close(_np(out), ref.detach().numpy(), 2e-4, 2e-5, name + " fwd")
        sc = max(1.0, float(x64.grad.abs().max()))
        assert_close(_np(xg.grad) / sc, x64.grad.numpy() / sc, 2e-4, 2e-5, name + " grad x")
        for k, v in layer.named_parameters():
            if params[k].grad is None:
                continue
            sc = max(1.0, float(params[k].grad.abs().max()))
            assert_close(_np(v.grad) / sc, params[k].grad.numpy() / sc, 2e-4, 2e-5, name + " grad " + k)

    inv = torch.where(deg > 0, 1.0 / deg.clamp(min=1), torch.zeros_like(deg))
    check(cxgnncomp.MyGCNConv(32, 48), lambda t, P: agg(t) @ P["lin.weight"].T + P["bias"], (pc, ic, n), "GCN sum")
    check(cxgnncomp.MyGCNConv(32, 16, normalize=True),
          lambda t, P: agg(t @ P["lin.weight"].T, inv[dst]) + P["bias"], (pc, ic, n), "GCN 1/deg, linear first")
    check(cxgnncomp.MySageConv(32, 48),
          lambda t, P: (agg(t) * inv[:, None]) @ P["lin_l.weight"].T + P["lin_l.bias"] + t @ P["lin_r.weight"].T,
          (pc, ic, n), "SAGE mean")
    check(cxgnncomp.MySageConv(32, 16),
          lambda t, P: agg(t @ P["lin_l.weight"].T + P["lin_l.bias"]) * inv[:, None] + t @ P["lin_r.weight"].T,
          (pc, ic, n), "SAGE mean, linear first")
    check(cxgnncomp.MySageConv(32, 40, root_weight=False, bias=False),
          lambda t, P: (agg(t) * inv[:, None]) @ P["lin_l.weight"].T, (pc, ic, n), "SAGE mean, no root, no bias")
    check(cxgnncomp.MyGINConv(32, 24),
          lambda t, P: (agg(t) * inv[:, None] + (1 + P["eps"]) * t) @ P["nn.weight"].T, (pc, ic, n), "GIN")

    def gat_ref(H, C, concat):
        def f(t, P):
            xs = (t @ P["lin_src"].T).view(-1, H, C)
            a_s = (xs * P["att_src"]).sum(-1)
            a_d = (xs * P["att_dst"]).sum(-1)
            ev = pyref.edge_softmax_opwise(ptr, idx, a_s, a_d, E, 0.2)
            out = agg(xs, None) * 0
            out = torch.zeros(n, H, C, dtype=t.dtype).index_add_(0, dst, xs[idx] * ev.unsqueeze(-1))
            out = out.view(-1, H * C) if concat else out.mean(dim=1)
            return out + P["bias"]
        return f
    check(cxgnncomp.MyGATConv(32, 16, heads=4, concat=True), gat_ref(4, 16, True), (pc, ic, n, n, E), "GAT 4 heads")
    check(cxgnncomp.MyGATConv(32, 16, heads=2, concat=False), gat_ref(2, 16, False), (pc, ic, n, n, E), "GAT mean heads")
    check(cxgnncomp.MyGATConv(32, 16, heads=1), gat_ref(1, 16, False), (pc, ic, n, n, E), "GAT 1 head, out<in")
    check(cxgnncomp.MyGATConv(32, 64, heads=1), gat_ref(1, 64, False), (pc, ic, n, n, E), "GAT 1 head, out>in")


@pytest.mark.parametrize("tables", ["dense", "pairs"])
def test_rgcn_conv_layer(tables, monkeypatch):
    import cxgnncomp
    from cxgnncomp_backend import _typed
    monkeypatch.setattr(_typed, "RGCN_PAIR_FILL_MAX", 2.0 if tables == "pairs" else -1.0)
    cxgnncomp.set_timers()
    ptr, idx, etype = _hetero(n=1500, e=20000, R=4, seed=8)
    n = ptr.shape[0] - 1
    torch.manual_seed(23)
    x = torch.randn(n, 32) / 8
    layer = cxgnncomp.MyRGCNConv(32, 32, 4).cuda()
    xg = x.cuda().requires_grad_(True)
    announce("MyRGCNConv")
    out = layer(xg, ptr.cuda(), idx.cuda(), etype.cuda(), n)
    out.sum().backward()
    torch.cuda.synchronize()
    w = layer.linear.detach().cpu()
    g = torch.ones(n, 32)
    deg = (ptr[1:] - ptr[:-1]).double().unsqueeze(-1)
    x64 = x.double().requires_grad_(True)
    ref = pyref.typed_linear_s2d_sort(x64, w.double(), ptr, idx, etype, n) / deg
    ref.backward(g.double())
    assert_close(_np(out), ref.detach().numpy(), RTOL, 2 * ATOL, "rgcn conv fwd")
    assert_close(_np(xg.grad), x64.grad.numpy(), RTOL, 2 * ATOL, "rgcn conv grad x")
    w64 = w.double().requires_grad_(True)
    (pyref.typed_linear_s2d_sort(x.double(), w64, ptr, idx, etype, n) / deg).backward(g.double())
    sc = float(w64.grad.abs().max())
    assert_close(_np(layer.linear.grad) / sc, w64.grad.numpy() / sc, RTOL, 2 * ATOL, "rgcn conv grad w")


def test_schedule_helpers_on_gpu_tensors():
    import cxgnncomp
    ptr, idx = _graph("powerlaw")
    want_ptr, want_target = oracle.neighbor_grouping(ptr.numpy(), 32)
    announce("neighbor_grouping on GPU tensors")
    gp, gt = cxgnncomp.neighbor_grouping(ptr.cuda(), 32)
    assert gp.is_cuda and np.array_equal(_np(gp), want_ptr) and np.array_equal(_np(gt), want_target)
    flag = torch.rand(ptr.shape[0] - 1) < 0.2
    a = cxgnncomp.remove_from_graph(ptr.cuda(), idx.cuda(), flag.cuda())
    b = cxgnncomp.remove_from_graph(ptr, idx, flag)
    assert torch.equal(a[0].cpu(), b[0]) and torch.equal(a[1].cpu(), b[1])


@pytest.mark.parametrize("heads,channels", [(4, 64), (1, 128), (2, 16), (3, 10)])
def test_head_dot_op(heads, channels):
    """HeadDotOP == (x * att).sum(-1) with the gradients autograd gives that expression."""
    from cxgnncomp.graph_conv import HeadDotOP
    torch.manual_seed(heads * 100 + channels)
    n = 5000
    x = torch.randn(n, heads, channels) / channels ** 0.5
    att = torch.randn(1, heads, channels)
    g = torch.randn(n, heads) / n ** 0.5
    xr, ar = x.double().requires_grad_(True), att.double().requires_grad_(True)
    ((xr * ar).sum(-1) * g.double()).sum().backward()
    xc, ac = x.cuda().requires_grad_(True), att.cuda().requires_grad_(True)
    announce("HeadDotOP H=%d C=%d" % (heads, channels))
    out = HeadDotOP.apply(xc, ac)
    out.backward(g.cuda())
    assert_close(_np(out), (x.double() * att.double()).sum(-1).numpy(), RTOL, ATOL, "head dot")
    assert_close(_np(xc.grad), xr.grad.numpy(), RTOL, ATOL, "head dot grad x")
    assert_close(_np(ac.grad), ar.grad.numpy(), RTOL, 2 * ATOL, "head dot grad att")
    # host tensors take the upstream expression
    assert torch.allclose(HeadDotOP.apply(x, att), (x * att).sum(-1))


@pytest.mark.parametrize("k,n", [(128, 256), (256, 256), (256, 40), (300, 64), (30, 16), (64, 7)])
@pytest.mark.parametrize("rows", [1, 5000, 70001])
def test_linear_op_matches_torch(k, n, rows):
    """The conv layers' linear: forward and input gradient from the library GEMM, weight
    gradient from the typed weight-gradient kernel (one launch per 128 input columns), with
    the library GEMM for shapes it does not take.  Reference: F.linear differentiated in
    double precision; 1e-4 relative / 2e-5 absolute on values scaled to O(1)."""
    from cxgnncomp.graph_conv import linear
    torch.manual_seed(k * n + rows)
    x = torch.randn(rows, k)
    w = torch.randn(n, k) / k ** 0.5
    b = torch.randn(n)
    g = torch.randn(rows, n) / max(1.0, rows ** 0.5)
    xd, wd, bd = (t.double().requires_grad_(True) for t in (x, w, b))
    (torch.nn.functional.linear(xd, wd, bd) * g.double()).sum().backward()
    xc, wc, bc = (t.cuda().requires_grad_(True) for t in (x, w, b))
    announce("linear op k=%d n=%d rows=%d" % (k, n, rows))
    out = linear(xc, wc, bc)
    (out * g.cuda()).sum().backward()
    torch.cuda.synchronize()
    ref = torch.nn.functional.linear(xd, wd, bd).detach()
    assert_close(out.detach().cpu().numpy(), ref.numpy(), 1e-4, 2e-5, "linear out")
    for got, want, name in ((xc.grad, xd.grad, "grad x"), (wc.grad, wd.grad, "grad w"), (bc.grad, bd.grad, "grad b")):
        assert got.shape == want.shape
        scale = max(1.0, float(want.abs().max()))
        assert_close(got.cpu().numpy() / scale, want.numpy() / scale, 1e-4, 2e-5, name)


@pytest.mark.parametrize("widths", [(24, 40), (40, 24)])
def test_sage_layer_on_a_row_prefix(widths):
    """MySageConv on a sampled-batch layer: num_node destination rows over more source rows
    (the root term reads x[:num_node]); output, input gradient and every parameter gradient
    against the float64 composition, and a frozen input (no input gradient asked for)."""
    import cxgnncomp
    torch.manual_seed(4)
    n_src, n_dst, fin, fout = 900, 300, widths[0], widths[1]
    deg = torch.randint(0, 9, (n_dst,))
    deg[5] = 0
    ptr = torch.zeros(n_dst + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(deg, 0)
    E = int(ptr[-1])
    idx = torch.randint(0, n_src, (E,))
    dst = torch.repeat_interleave(torch.arange(n_dst), deg)
    x = torch.randn(n_src, fin)
    layer = cxgnncomp.MySageConv(fin, fout).cuda()
    xg = x.cuda().requires_grad_(True)
    announce("SageLayerOP prefix rows %s" % (widths,))
    out = layer(xg, ptr.cuda(), idx.cuda(), n_dst)
    w = torch.randn(n_dst, fout)
    (out * w.cuda()).sum().backward()
    torch.cuda.synchronize()
    P = {k: v.detach().double().cpu().requires_grad_(True) for k, v in layer.named_parameters()}
    x64 = x.double().requires_grad_(True)
    inv = torch.where(deg > 0, 1.0 / deg.clamp(min=1).double(), torch.zeros(n_dst, dtype=torch.float64))

    def mean_aggr(t):
        return torch.zeros(n_dst, t.shape[1], dtype=t.dtype).index_add_(0, dst, t[idx]) * inv[:, None]
    if fin > fout:
        ref = mean_aggr(x64 @ P["lin_l.weight"].T + P["lin_l.bias"])
    else:
        ref = mean_aggr(x64) @ P["lin_l.weight"].T + P["lin_l.bias"]
    ref = ref + x64[:n_dst] @ P["lin_r.weight"].T
    (ref * w.double()).sum().backward()
    assert_close(_np(out), ref.detach().numpy(), 2e-4, 2e-5, "fwd")
    assert_close(_np(xg.grad), x64.grad.numpy(), 2e-4, 2e-5, "grad x")
    for k, v in layer.named_parameters():
        sc = max(1.0, float(P[k].grad.abs().max()))
        assert_close(_np(v.grad) / sc, P[k].grad.numpy() / sc, 2e-4, 2e-5, "grad " + k)
    # frozen input: parameter gradients only
    layer.zero_grad()
    out2 = layer(x.cuda(), ptr.cuda(), idx.cuda(), n_dst)
    (out2 * w.cuda()).sum().backward()
    assert torch.equal(out2, out)
    for k, v in layer.named_parameters():
        sc = max(1.0, float(P[k].grad.abs().max()))
        assert_close(_np(v.grad) / sc, P[k].grad.numpy() / sc, 2e-4, 2e-5, "frozen input, grad " + k)


def _gat_layer_on_a_row_prefix(H, C, concat, max_deg, fin, frozen=False):
    import cxgnncomp
    cxgnncomp.set_timers()               # MyGATConv brackets its phases with TimerOP, as upstream
    torch.manual_seed(6)
    n_all, n_src, n_dst = 700, 600, 200
    deg = torch.randint(0, max_deg, (n_dst,))
    deg[3] = 0
    ptr = torch.zeros(n_dst + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(deg, 0)
    E = int(ptr[-1])
    idx = torch.randint(0, n_src, (E,))
    dst = torch.repeat_interleave(torch.arange(n_dst), deg)
    x = torch.randn(n_all, fin) / (fin / 24) ** 0.5
    layer = cxgnncomp.MyGATConv(fin, C, heads=H, concat=concat).cuda()
    with torch.no_grad():
        layer.bias.normal_()
    xg = x.cuda().requires_grad_(not frozen)
    announce("GatLayerOP prefix rows concat=%s H=%d C=%d in=%d E=%d frozen=%s" % (concat, H, C, fin, E, frozen))
    out = layer(xg, ptr.cuda(), idx.cuda(), n_dst, n_src, E)
    w = torch.randn(*out.shape)
    (out * w.cuda()).sum().backward()
    torch.cuda.synchronize()
    P = {k: v.detach().double().cpu().requires_grad_(True) for k, v in layer.named_parameters()}
    x64 = x.double().requires_grad_(True)
    xs = (x64[:n_src] @ P["lin_src"].T).view(-1, H, C)
    a_s = (xs * P["att_src"]).sum(-1)
    a_d = (xs[:n_dst] * P["att_dst"]).sum(-1)
    ev = pyref.edge_softmax_opwise(ptr, idx, a_s, a_d, E, 0.2)
    ref = torch.zeros(n_dst, H, C, dtype=torch.float64).index_add_(0, dst, xs[idx] * ev.unsqueeze(-1))
    ref = (ref.view(-1, H * C) if concat else ref.mean(dim=1)) + P["bias"]
    (ref * w.double()).sum().backward()
    assert out.shape == ref.shape
    assert_close(_np(out), ref.detach().numpy(), 2e-4, 2e-5, "fwd")
    if frozen:
        assert xg.grad is None
    else:
        assert xg.grad.shape == x.shape and float(xg.grad[n_src:].abs().max()) == 0.0
        sc = max(1.0, float(x64.grad.abs().max()))
        assert_close(_np(xg.grad) / sc, x64.grad.numpy() / sc, 2e-4, 2e-5, "grad x")
    for k, v in layer.named_parameters():
        sc = max(1.0, float(P[k].grad.abs().max()))
        assert_close(_np(v.grad) / sc, P[k].grad.numpy() / sc, 2e-4, 2e-5, "grad " + k)


@pytest.mark.parametrize("heads_channels", [(4, 8), (4, 64), (2, 32), (8, 16)])
@pytest.mark.parametrize("concat", [True, False])
@pytest.mark.parametrize("max_deg", [12, 40])
def test_gat_layer_on_a_row_prefix(concat, heads_channels, max_deg):
    """MyGATConv (several heads, one autograd node on CUDA) on a sampled-batch layer: num_dst
    destination rows over num_src source rows of a longer x; output and every gradient against
    the float64 composition of the upstream expressions.  With about 20 edges per row and an
    input of 24 columns against 64 or more of transformed features the layer aggregates the
    input rows under the H edge weights and transforms afterwards; with about 6 it aggregates
    the transformed rows."""
    H, C = heads_channels       # 4 x 64 = 256 floats per row: the backward pass with the fused edge products
    _gat_layer_on_a_row_prefix(H, C, concat, max_deg, 24)


@pytest.mark.parametrize("fin,C", [(24, 64), (24, 16), (24, 24), (256, 512), (256, 256), (128, 256), (100, 128), (30, 64),
                                   (256, 128), (256, 100)])
@pytest.mark.parametrize("frozen", [False, True])
def test_gat_single_head_layer_on_a_row_prefix(fin, C, frozen):
    """MyGATConv with one head (upstream's forward_1, cxgnncomp/graph_conv.py:498-547) on the same
    layer node: an input narrower than the output is aggregated first and transformed afterwards,
    forward and backward on rows of `in` floats (from 96 columns on the backward pass over the
    reversed graph also leaves the edge-value gradient; 30 columns are not a multiple of 4 and
    take the transformed rows); otherwise the transformed rows are aggregated (with the fused
    backward pass from 96 output columns on).  Output and every gradient against float64, also
    with an input that needs no gradient."""
    _gat_layer_on_a_row_prefix(1, C, False, 40, fin, frozen)


@pytest.mark.parametrize("opname", ["RGCNOP", "RGCNOP2", "TypedLinearS2DSort"])
def test_rgcn_ops_on_a_graph_without_edges(opname):
    """No edge at all: zeros out, zero gradients, no launch on empty pair tables."""
    import cxgnncomp
    from cxgnncomp import graph_conv
    cxgnncomp.set_timers()
    n, K, N, R = 70, 16, 8, 3
    ptr = torch.zeros(n + 1, dtype=torch.int64).cuda()
    idx = torch.zeros(0, dtype=torch.int64).cuda()
    etype = torch.zeros(0, dtype=torch.int32).cuda()
    x = torch.randn(n, K).cuda().requires_grad_(True)
    w = torch.randn(R, K, N).cuda().requires_grad_(True)
    announce("%s without edges" % opname)
    if opname == "TypedLinearS2DSort":
        out = cxgnncomp.TypedLinearS2DSort(x, w, ptr, idx, etype, n)
    else:
        out = getattr(graph_conv, opname).apply(x, w, ptr, idx, etype, n)
    out.sum().backward()
    torch.cuda.synchronize()
    assert out.shape == (n, N) and float(out.detach().abs().max()) == 0.0
    assert float(x.grad.abs().max()) == 0.0 and float(w.grad.abs().max()) == 0.0
